"""``update_out_and_lse`` for unchanged generated code, with the merges of a step deferred to ONE fold.

The generated chunk loop calls ``update_out_and_lse`` once per chunk (utils/flash_attn_dsl.py:176-177 and the
five sibling templates) and then stores ``_out.to(q.dtype)`` and ``_lse.squeeze(dim=-1).transpose(1, 2)``
(utils/flash_attn_dsl.py:178-179).  Run literally, the fp32 accumulator travels through memory once per chunk.
The fold is associative, so the lazy variant of this module hands the generated code two light handles instead
of accumulator tensors; each call only records ``(block_out, block_lse, first row)``.  When the epilogue
expressions run, the handles fold everything recorded with one ``merge_many`` call (every bf16 block output
read once) and return the finished bf16 output and ``(B, H, S)`` LSE.

Anything else the caller does with a handle -- an attribute the epilogue does not use, a ``torch`` function, a
``slice_`` that is not "rows from a on", more blocks than one fold takes, a dtype other than bfloat16 -- makes
the handle compute the accumulators with the literal chain of merges (``merge.update_out_and_lse``) and behave
like the resulting tensor, so the lazy namespace never changes what generated code computes, only how often the
accumulator moves.

Install with ``exec(text, mercury_artifact_amd.namespace(lazy_merge=True))``.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import merge as _merge

__all__ = ["update_out_and_lse_lazy", "LazyOut", "LazyLse"]


class _Pending:
    """The merges recorded so far for one pair of handles."""

    def __init__(self, blocks: List[Tuple[torch.Tensor, torch.Tensor, int]]):
        self.blocks = blocks            # (block_out, block_lse, first sequence row covered)
        self.chain = None               # (out fp32 (B,Sq,Hq,D), lse fp32 (B,Sq,Hq,1)) once the literal chain ran
        self.folded = None              # (out bf16 (B,Sq,Hq,D), lse fp32 (B,Hq,Sq)) once the one-pass fold ran

    @property
    def shape(self):
        return tuple(self.blocks[0][0].shape)

    def foldable(self) -> bool:
        if self.chain is not None or len(self.blocks) > _merge.MAX_MERGE_MANY:
            return False
        first = self.blocks[0][0]
        ss, sh = first.stride(1), first.stride(2)
        for bo, bl, _ in self.blocks:
            if bo.dtype != torch.bfloat16 or bo.stride(3) != 1 or (bo.stride(1), bo.stride(2)) != (ss, sh):
                return False
            if bl.dtype != torch.float32 or not bl.is_contiguous():
                return False
        return first.shape[-1] % 8 == 0 and first.shape[-1] <= 256

    def fold(self):
        if self.folded is None:
            B, Sq, Hq, D = self.shape
            dev = self.blocks[0][0].device
            out = torch.empty((B, Sq, Hq, D), dtype=torch.bfloat16, device=dev)
            lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=dev)
            _merge.merge_many([b[0] for b in self.blocks], [b[1] for b in self.blocks], out, lse,
                              row_begin=[b[2] for b in self.blocks])
            self.folded = (out, lse)
        return self.folded

    def run_chain(self):
        """The literal sequence of merges, as merge.update_out_and_lse performs them."""
        if self.chain is None:
            out = lse = None
            for bo, bl, begin in self.blocks:
                sl = None if begin == 0 else (slice(None), slice(begin, None))
                out, lse = _merge.update_out_and_lse(out, lse, bo, bl, slice_=sl)
            self.chain = (out, lse)
        return self.chain


def _real(x):
    """Handles replaced by the tensors they stand for (inside lists and tuples too)."""
    if isinstance(x, _TensorLike):
        return x.materialize()
    if isinstance(x, (list, tuple)):
        return type(x)(_real(y) for y in x)
    return x


class _TensorLike:
    """Behaves like the tensor ``materialize()`` returns for everything a subclass does not answer lazily:
    attributes and methods, indexing, torch functions, and the operators Python looks up on the type
    (arithmetic, comparisons, unary, in-place, ``len`` / ``iter`` / ``bool`` / ``float``)."""

    def materialize(self) -> torch.Tensor:
        raise NotImplementedError

    def __getattr__(self, name):
        return getattr(self.materialize(), name)

    def __getitem__(self, item):
        return self.materialize()[_real(item)]

    def __setitem__(self, item, value):
        self.materialize()[_real(item)] = _real(value)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        return func(*_real(args), **{k: _real(v) for k, v in (kwargs or {}).items()})

    __hash__ = object.__hash__


def _install_operators():
    def binary(name):
        def op(self, other):
            return getattr(self.materialize(), name)(_real(other))
        op.__name__ = name
        return op

    def inplace(name):
        def op(self, other):
            getattr(self.materialize(), name)(_real(other))
            return self                      # the handle goes on standing for the tensor that was updated
        op.__name__ = name
        return op

    def unary(name):
        def op(self):
            return getattr(self.materialize(), name)()
        op.__name__ = name
        return op

    arithmetic = ["add", "sub", "mul", "truediv", "floordiv", "mod", "pow", "matmul", "and", "or", "xor",
                  "lshift", "rshift"]
    for base in arithmetic:
        setattr(_TensorLike, f"__{base}__", binary(f"__{base}__"))
        setattr(_TensorLike, f"__r{base}__", binary(f"__r{base}__"))
        setattr(_TensorLike, f"__i{base}__", inplace(f"__i{base}__"))
    for base in ["lt", "le", "gt", "ge", "eq", "ne"]:
        setattr(_TensorLike, f"__{base}__", binary(f"__{base}__"))
    for base in ["neg", "pos", "abs", "invert", "len", "iter", "bool", "float", "int", "index"]:
        setattr(_TensorLike, f"__{base}__", unary(f"__{base}__"))


_install_operators()


class _Handle(_TensorLike):
    """Stands for one of the two accumulators; everything it is not asked lazily goes to the real tensor."""

    _which = 0

    def __init__(self, pending: _Pending):
        object.__setattr__(self, "_p", pending)

    def materialize(self) -> torch.Tensor:
        return self._p.run_chain()[self._which]

    @property
    def dtype(self):
        return torch.float32

    @property
    def device(self):
        return self._p.blocks[0][0].device


class LazyOut(_Handle):
    _which = 0

    @property
    def shape(self):
        return torch.Size(self._p.shape)

    def to(self, *args, **kwargs):
        """``_out.to(q.dtype)`` of the epilogue: a plain cast to bfloat16 is answered by the fold."""
        dtype = kwargs.get("dtype", args[0] if len(args) == 1 and not kwargs else None)
        plain = (len(args) == 1 and not kwargs) or (not args and set(kwargs) == {"dtype"})
        if plain and dtype == torch.bfloat16 and self._p.foldable():
            return self._p.fold()[0]
        return self.materialize().to(*args, **kwargs)


class _SqueezedLse(_TensorLike):
    """``_lse.squeeze(dim=-1)``: (B, Sq, Hq) in the reference; only ``transpose(1, 2)`` is answered lazily."""

    def __init__(self, pending: _Pending):
        object.__setattr__(self, "_p", pending)

    def materialize(self) -> torch.Tensor:
        return self._p.run_chain()[1].squeeze(dim=-1)

    def transpose(self, dim0, dim1):
        if sorted((dim0 % 3, dim1 % 3)) == [1, 2] and self._p.foldable():
            return self._p.fold()[1]
        return self.materialize().transpose(dim0, dim1)


class LazyLse(_Handle):
    _which = 1

    @property
    def shape(self):
        B, Sq, Hq, _ = self._p.shape
        return torch.Size((B, Sq, Hq, 1))

    def squeeze(self, *args, **kwargs):
        dim = kwargs.get("dim", args[0] if len(args) == 1 and not kwargs else None)
        if dim in (-1, 3) and len(args) + len(kwargs) == 1:
            return _SqueezedLse(self._p)
        return self.materialize().squeeze(*args, **kwargs)


def _first_row(slice_, Sq: int) -> Optional[int]:
    """The row ``a`` if ``slice_`` selects "all batches, rows a.." of a (B, Sq, ...) tensor, else None."""
    if slice_ is None:
        return 0
    if not isinstance(slice_, tuple) or not 1 <= len(slice_) <= 2:
        return None
    if slice_[0] != slice(None) and slice_[0] != slice(None, None, None):
        return None
    if len(slice_) == 1:
        return 0
    rows = slice_[1]
    if not isinstance(rows, slice) or rows.step not in (None, 1) or rows.stop not in (None, Sq):
        return None
    a = 0 if rows.start is None else rows.start
    return a if isinstance(a, int) and 0 <= a <= Sq else None


def update_out_and_lse_lazy(out, lse, block_out: torch.Tensor, block_lse: torch.Tensor, slice_=None):
    """``update_out_and_lse`` (utils/flash_attn_dsl.py:51-71) that records instead of merging; see the module
    text.  Same call signature, same errors, same functional / in-place behaviour: without ``slice_`` the
    result is a new pair of handles and the arguments keep standing for the state before the call; with
    ``slice_`` the arguments themselves are updated and returned."""
    if out is None:
        if slice_ is not None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        pending = _Pending([(block_out, block_lse, 0)])
        return LazyOut(pending), LazyLse(pending)
    lazy = isinstance(out, LazyOut) and isinstance(lse, LazyLse) and out._p is lse._p and out._p.chain is None
    if lazy:
        pending = out._p
        B, Sq, Hq, D = pending.shape
        begin = _first_row(slice_, Sq)
        fits = (begin is not None and tuple(block_out.shape) == (B, Sq - begin, Hq, D)
                and len(pending.blocks) < _merge.MAX_MERGE_MANY and pending.folded is None)
        if fits:
            if slice_ is None:
                fresh = _Pending(pending.blocks + [(block_out, block_lse, 0)])
                return LazyOut(fresh), LazyLse(fresh)
            pending.blocks.append((block_out, block_lse, begin))
            return out, lse
    # the literal merge on real accumulators (materialised from what was recorded, if anything was)
    if isinstance(out, _Handle) or isinstance(lse, _Handle):
        real_out = out.materialize() if isinstance(out, _Handle) else out
        real_lse = lse.materialize() if isinstance(lse, _Handle) else lse
        if slice_ is not None:
            _merge.update_out_and_lse(real_out, real_lse, block_out, block_lse, slice_=slice_)
            return out, lse          # in place: the handles now stand for the updated tensors
        return _merge.update_out_and_lse(real_out, real_lse, block_out, block_lse)
    return _merge.update_out_and_lse(out, lse, block_out, block_lse, slice_=slice_)
