"""Timing harness with the contract of Mercury's schedule search (mercury/search/bench.py:15-86), so that the
search can time candidate schedules on this package's kernels.

The reference's ``bench_program`` lowers an IR program to PyTorch text, ``exec``s it in a namespace that
already holds the operator names, allocates one tensor per I/O buffer (zeros for outputs, N(0,1) for
inputs), runs ``num_iter`` warm-up calls and ``num_iter`` timed calls between two device events, and returns
``(iterations per second, seconds, bytes of buffer memory)``.  Here:

* :func:`bench_callable` is that timing protocol for a function that already exists;
* :func:`bench_program` is the whole thing: lowering (the reference's generator, imported lazily because it is
  not part of this package, or any :class:`Lowering` the caller passes), ``exec`` into a namespace filled with
  :func:`mercury_artifact_amd.namespace`, buffer allocation, timing.
"""
from __future__ import annotations

import os
from typing import Callable, Dict, Iterable, NamedTuple, Optional, Tuple

import torch

__all__ = ["bench_callable", "bench_program", "Lowering", "mercury_lowering"]


def bench_callable(func: Callable[..., object], kwargs: Dict[str, object], num_iter: int = 100,
                   memory_bytes: Optional[int] = None, log: bool = False) -> Tuple[float, float, int]:
    """``num_iter`` warm-up calls, then ``num_iter`` calls of ``func(**kwargs)`` between two device events on the
    current stream.  Returns (iterations per second, seconds, bytes), bytes being ``memory_bytes`` or, if not
    given, the size of the tensors in ``kwargs``."""
    if not torch.cuda.is_available():
        raise RuntimeError("bench_callable needs a GPU")
    if num_iter <= 0:
        raise ValueError("num_iter must be positive")
    if memory_bytes is None:
        memory_bytes = sum(v.numel() * v.element_size() for v in kwargs.values() if isinstance(v, torch.Tensor))
    with torch.no_grad():
        for _ in range(num_iter):
            func(**kwargs)
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for _ in range(num_iter):
            func(**kwargs)
        end.record()
    torch.cuda.synchronize()
    seconds = begin.elapsed_time(end) / 1e3
    if log:
        print(f"Memory cost: {memory_bytes / 1024 / 1024:.2f} MB")
        print(f"{num_iter / seconds:.3f} iter/s, {seconds:.3f} sec")
    return num_iter / seconds, seconds, int(memory_bytes)


class Lowering(NamedTuple):
    """The four things ``bench_program`` needs from an IR: in the reference they are
    ``mercury.ir.loop_eliminating.eliminate_loops``, ``mercury.backend.pytorch.codegen.generate_pytorch_code``,
    ``program.visit(mercury.ir.utils.get_io_buffers)`` and ``mercury.ir.calculate_memory.get_buffer_size``."""
    eliminate_loops: Callable[[object], object]
    generate_code: Callable[[object], str]       # -> source text defining a function called program.name
    io_buffers: Callable[[object], Iterable]     # -> objects with .tensor (argument name), .shape, .dtype, .write
    buffer_bytes: Callable[[object], int]


def mercury_lowering() -> Lowering:
    """The reference's own lowering, imported on demand (its package is not part of this one)."""
    try:
        from mercury.backend.pytorch.codegen import generate_pytorch_code
        from mercury.ir.calculate_memory import get_buffer_size
        from mercury.ir.loop_eliminating import eliminate_loops
        from mercury.ir.utils import get_io_buffers
    except ImportError as exc:
        raise ImportError("bench_program lowers Mercury IR and needs the `mercury` package on the path (or a "
                          "`lowering` argument); use bench_callable for a function that is already generated") from exc
    return Lowering(eliminate_loops, generate_pytorch_code, lambda program: program.visit(get_io_buffers),
                    get_buffer_size)


def bench_program(program, namespace: Optional[dict] = None, num_iter: int = 100,
                  kwargs: Optional[dict] = None, log: bool = True, lowering: Optional[Lowering] = None,
                  lazy_merge: bool = True) -> Tuple[float, float, int]:
    """Counterpart of the reference's ``bench_program`` (mercury/search/bench.py:15-86): lower ``program`` to
    source text, ``exec`` it in a namespace filled with this package's operators (``lazy_merge`` as in
    :func:`mercury_artifact_amd.namespace`), allocate one tensor per I/O buffer on this rank's device (zeros
    for the buffers the program writes, N(0,1) for the others), and time the function ``program.name`` with
    :func:`bench_callable`.  ``lowering`` defaults to the reference's generator (:func:`mercury_lowering`)."""
    import torch.distributed as dist

    from . import namespace as _names

    low = lowering if lowering is not None else mercury_lowering()
    rank = dist.get_rank() if dist.is_initialized() else 0
    device = torch.device(f"cuda:{int(os.getenv('LOCAL_RANK', rank))}")
    torch.cuda.set_device(device)
    ns = dict(namespace) if namespace is not None else {}
    ns.update(_names(lazy_merge=lazy_merge))
    low.eliminate_loops(program)
    code = low.generate_code(program)
    if rank == 0 and log:
        print(code)
    exec(code, ns)
    func = ns[program.name]
    call = dict(kwargs) if kwargs is not None else {}
    for buffer in low.io_buffers(program):
        make = torch.zeros if buffer.write else torch.randn
        call[buffer.tensor] = make(tuple(buffer.shape), device=device, dtype=buffer.dtype)
    return bench_callable(func, call, num_iter, memory_bytes=low.buffer_bytes(program), log=log and rank == 0)
