"""Merge helpers the generated ring code calls by bare name.

Same names, arguments and error behaviour as utils/flash_attn_dsl.py:14-71, 293-305 of the
reference; the arithmetic runs in the gfx950 kernels behind mhip_lse_merge / mhip_flash_reduce /
mhip_pack_reduce.  GPU tensors only.
"""
from __future__ import annotations

import inspect
from functools import cache
from typing import Optional, Sequence, Tuple

import torch

from . import _native as N
from .schedule import LocalGroup

__all__ = ["get_default_args", "update_out_and_lse", "_update_out_and_lse", "flash_reduce",
           "pack_block", "unpack_into", "merge_into", "merge_many", "grad_accumulate", "update_out_and_lse_collective", "add_collective",
           "LocalGroup"]


@cache
def _keyword_defaults(func):
    """Name -> default of every parameter that can be passed by keyword position-or-name; ``None`` where the
    signature gives no default; ``softcap`` pinned to 0.0."""
    named = (inspect.Parameter.POSITIONAL_ONLY, inspect.Parameter.POSITIONAL_OR_KEYWORD)
    table = {}
    for name, par in inspect.signature(func).parameters.items():
        if par.kind in named:
            table[name] = None if par.default is inspect.Parameter.empty else par.default
    if "softcap" in table:
        table["softcap"] = 0.0
    return table


def get_default_args(func):
    """Same contract as utils/flash_attn_dsl.py:14-29: keyword -> default of ``func`` (or of the Python function
    a ``torch.library`` custom op was created from), parameters without a default mapped to ``None`` and
    ``softcap`` forced to 0.0.  The dict is cached per function: the caller copies it before updating it, as the
    generated code does."""
    return _keyword_defaults(func if inspect.isfunction(func) else func._init_fn)


def _row_strides(t: torch.Tensor):
    return t.stride(0), t.stride(1), t.stride(2)


def merge_into(acc_out: Optional[torch.Tensor], acc_lse: Optional[torch.Tensor],
               block_out: torch.Tensor, block_lse: torch.Tensor,
               dst_out: Optional[torch.Tensor], dst_lse: Optional[torch.Tensor],
               final_out: Optional[torch.Tensor] = None, final_lse: Optional[torch.Tensor] = None) -> None:
    """One call of mhip_lse_merge.  acc (B,Sq,Hq,D)/(B,Sq,Hq,1) fp32 or None for the first block,
    block_out (B,Sq,Hq,D) bf16, block_lse (B,Hq,Sq) fp32, dst like acc (may be acc itself),
    final_out (B,Sq,Hq,D) bf16 contiguous and final_lse (B,Hq,Sq) fp32 contiguous or None."""
    N.require_cuda(acc_out, acc_lse, block_out, block_lse, dst_out, dst_lse, final_out, final_lse)
    B, Sq, Hq, D = block_out.shape
    if block_out.dtype != torch.bfloat16 or block_out.stride(-1) != 1:
        raise RuntimeError("block_out must be bfloat16 with a contiguous last dimension")
    if block_lse.shape != (B, Hq, Sq) or block_lse.dtype != torch.float32 or block_lse.stride(2) != 1:
        raise RuntimeError("block_lse must be float32 (B, Hq, Sq) with contiguous rows")
    for name, o, l in (("acc", acc_out, acc_lse), ("dst", dst_out, dst_lse)):
        if o is None:
            continue
        if o.shape != (B, Sq, Hq, D) or l.shape != (B, Sq, Hq, 1):
            raise RuntimeError(f"{name} shapes {tuple(o.shape)} / {tuple(l.shape)} do not match the block")
        if o.dtype != torch.float32 or l.dtype != torch.float32 or o.stride(-1) != 1:
            raise RuntimeError(f"{name} must be float32 with a contiguous last dimension")
    if final_out is not None:
        if not (final_out.is_contiguous() and final_lse.is_contiguous()):
            raise RuntimeError("final_out / final_lse must be contiguous")
        if final_out.shape != (B, Sq, Hq, D) or final_lse.shape != (B, Hq, Sq):
            raise RuntimeError("final_out / final_lse shapes do not match the block")
    z3 = (0, 0, 0)
    with torch.cuda.device(block_out.device):
        code = N.lib().mhip_lse_merge(
            N.ptr(acc_out), N.ptr(acc_lse), N.ptr(block_out), N.ptr(block_lse),
            N.ptr(dst_out), N.ptr(dst_lse), N.ptr(final_out), N.ptr(final_lse),
            B, Sq, Hq, D,
            *(z3 if acc_out is None else _row_strides(acc_out)),
            *(z3 if acc_lse is None else _row_strides(acc_lse)),
            *_row_strides(block_out), block_lse.stride(0), block_lse.stride(1),
            *(z3 if dst_out is None else _row_strides(dst_out)),
            *(z3 if dst_lse is None else _row_strides(dst_lse)),
            N.stream_of(block_out))
    N.check(code, "mhip_lse_merge")


MAX_MERGE_MANY = 64


def merge_many(block_outs: Sequence[torch.Tensor], block_lses: Sequence[torch.Tensor],
               final_out: torch.Tensor, final_lse: torch.Tensor,
               row_begin: Optional[Sequence[int]] = None) -> None:
    """All block results of a step folded by one call of mhip_lse_merge_many: what the chain of
    ``update_out_and_lse`` calls of the chunk loop plus the stores of utils/flash_attn_dsl.py:178-179
    compute (the fold is associative), reading every bf16 block output once.  Block i covers the sequence
    rows ``row_begin[i]:`` (default 0, i.e. all rows; the ``slice_`` merges of a zigzag schedule pass the
    start of their row range): block_outs[i] (B, Sq - row_begin[i], Hq, D) bf16 with contiguous heads,
    block_lses[i] (B, Hq, Sq - row_begin[i]) fp32 contiguous, at most ``MAX_MERGE_MANY`` blocks;
    final_out (B,Sq,Hq,D) bf16 and final_lse (B,Hq,Sq) fp32, both contiguous, are written."""
    import ctypes

    n = len(block_outs)
    if n != len(block_lses) or not 1 <= n <= MAX_MERGE_MANY:
        raise RuntimeError(f"merge_many takes 1..{MAX_MERGE_MANY} blocks with one lse each")
    begins = [0] * n if row_begin is None else [int(x) for x in row_begin]
    if len(begins) != n:
        raise RuntimeError("row_begin needs one entry per block")
    N.require_cuda(*block_outs, *block_lses, final_out, final_lse)
    B, Sq, Hq, D = final_out.shape
    if final_out.dtype != torch.bfloat16 or not final_out.is_contiguous():
        raise RuntimeError("final_out must be contiguous bfloat16 (B,Sq,Hq,D)")
    if final_lse.shape != (B, Hq, Sq) or final_lse.dtype != torch.float32 or not final_lse.is_contiguous():
        raise RuntimeError("final_lse must be contiguous float32 (B,Hq,Sq)")
    ss, sh = block_outs[0].stride(1), block_outs[0].stride(2)
    for bo, bl, sb in zip(block_outs, block_lses, begins):
        if not 0 <= sb <= Sq:
            raise RuntimeError("row_begin outside the sequence")
        if bo.shape != (B, Sq - sb, Hq, D) or bo.dtype != torch.bfloat16:
            raise RuntimeError("block outputs must be bfloat16 (B, Sq - row_begin, Hq, D)")
        if bo.stride(3) != 1 or (bo.stride(1), bo.stride(2)) != (ss, sh):
            raise RuntimeError("block outputs need a contiguous head dimension and common row / head strides")
        if bl.shape != (B, Hq, Sq - sb) or bl.dtype != torch.float32 or not bl.is_contiguous():
            raise RuntimeError("block lse must be contiguous float32 (B, Hq, Sq - row_begin)")
    if B * Sq * Hq == 0:
        return
    # a block that starts past the last row contributes nothing (and has no memory to point at)
    keep = [i for i in range(n) if begins[i] < Sq]
    if not keep:
        raise RuntimeError("merge_many needs at least one block that covers a row")
    block_outs, block_lses = [block_outs[i] for i in keep], [block_lses[i] for i in keep]
    begins, n = [begins[i] for i in keep], len(keep)
    outs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in block_outs])
    lses = (ctypes.c_void_p * n)(*[t.data_ptr() for t in block_lses])
    sbs = (ctypes.c_int64 * n)(*[t.stride(0) for t in block_outs])
    rbs = (ctypes.c_int * n)(*begins)
    with torch.cuda.device(final_out.device):
        code = N.lib().mhip_lse_merge_many(outs, lses, sbs, rbs, n, N.ptr(final_out), N.ptr(final_lse),
                                           B, Sq, Hq, D, ss, sh, N.stream_of(final_out))
    N.check(code, "mhip_lse_merge_many")


def _update_out_and_lse(out: torch.Tensor, lse: torch.Tensor, block_out: torch.Tensor,
                        block_lse: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """utils/flash_attn_dsl.py:31-49 -- functional: returns new (out, lse), inputs untouched."""
    block_out = block_out if block_out.dtype == torch.bfloat16 else block_out.to(torch.bfloat16)
    new_out = torch.empty(out.shape, dtype=torch.float32, device=out.device)
    new_lse = torch.empty(lse.shape, dtype=torch.float32, device=lse.device)
    merge_into(out, lse, block_out, block_lse, new_out, new_lse)
    return new_out, new_lse


def update_out_and_lse(out: Optional[torch.Tensor], lse: Optional[torch.Tensor],
                       block_out: torch.Tensor, block_lse: torch.Tensor, slice_=None,
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """utils/flash_attn_dsl.py:51-71.  First call (``out is None``) turns the block into the fp32
    accumulators; ``slice_`` merges into that sub-range of the accumulators in place; otherwise a
    functional merge."""
    first = out is None
    if first and slice_ is not None:
        raise RuntimeError("first update_out_and_lse should not pass slice_ args")      # the reference's message
    if first:                                         # the block becomes the fp32 accumulators: one cast kernel
        B, Sq, Hq, D = block_out.shape
        acc_out = torch.empty((B, Sq, Hq, D), dtype=torch.float32, device=block_out.device)
        acc_lse = torch.empty((B, Sq, Hq, 1), dtype=torch.float32, device=block_out.device)
        merge_into(None, None, block_out, block_lse, acc_out, acc_lse)
        return acc_out, acc_lse
    if slice_ is None:                                # functional: new accumulators
        return _update_out_and_lse(out, lse, block_out, block_lse)
    part_out, part_lse = out[slice_], lse[slice_]     # in place on the views the slice selects
    merge_into(part_out, part_lse, block_out, block_lse, part_out, part_lse)
    return out, lse


def flash_reduce(lhs: torch.Tensor, rhs: torch.Tensor) -> torch.Tensor:
    """utils/flash_attn_dsl.py:293-305 on packed ``[..., D+1]`` fp32 operands; returns a new tensor."""
    N.require_cuda(lhs, rhs)
    if lhs.shape != rhs.shape or lhs.dtype != torch.float32 or rhs.dtype != torch.float32:
        raise RuntimeError("flash_reduce takes two float32 tensors of one shape")
    lhs, rhs = lhs.contiguous(), rhs.contiguous()
    dst = torch.empty_like(lhs)
    W = lhs.shape[-1]
    rows = lhs.numel() // W if W else 0
    with torch.cuda.device(lhs.device):
        code = N.lib().mhip_flash_reduce(N.ptr(lhs), N.ptr(rhs), N.ptr(dst), rows, W - 1, N.stream_of(lhs))
    N.check(code, "mhip_flash_reduce")
    return dst


def _is_collective(op, name: str) -> bool:
    return op == name or getattr(op, "__name__", None) == name


def _tree_merge(src: torch.Tensor, row_max: torch.Tensor, dst: torch.Tensor, finish: bool) -> None:
    W = src.shape[-1]
    rows = src.numel() // W if W else 0
    with torch.cuda.device(src.device):
        code = N.lib().mhip_tree_merge(N.ptr(src), N.ptr(row_max), N.ptr(dst), rows, W - 1, int(finish),
                                       N.stream_of(src))
    N.check(code, "mhip_tree_merge")


def update_out_and_lse_collective(tensor: torch.Tensor, op, group: LocalGroup, dst: Optional[int] = None) -> None:
    """utils/flash_attn_dsl.py:307-324: merge the packed ``(out | lse)`` partial results of all ranks of
    ``group`` the tree-attention way (MAX of the lse, SUM of ``out * d`` and ``d``) and write the merged
    value into ``tensor`` in place.  ``op`` is ``dist.all_reduce`` or ``dist.reduce`` (the function or its
    name); with ``reduce`` only rank ``dst`` receives the result.  The per-rank arithmetic runs in two
    kernels (``mhip_tree_merge``); the collectives themselves are replayed over the operands of the group's ranks: one MAX
    over the lse columns and ONE SUM over the packed ``(out * d | d)`` terms."""
    reduce_to_one = _is_collective(op, "reduce")
    if not (reduce_to_one or _is_collective(op, "all_reduce")):
        raise RuntimeError("Unsupported collective op")
    peers = [p.contiguous() for p in group.operands(tensor)]
    N.require_cuda(tensor, *peers)
    for p in peers:
        if p.shape != tensor.shape or p.dtype != torch.float32:
            raise RuntimeError("all ranks contribute float32 tensors of one shape")
    row_max = peers[0][..., -1].contiguous()
    for p in peers[1:]:
        row_max = torch.maximum(row_max, p[..., -1])          # the MAX all-reduce
    total = None
    for p in peers:
        term = torch.empty_like(p)
        _tree_merge(p, row_max, term, finish=False)
        total = term if total is None else total.add_(term)   # the SUM all-reduce
    if reduce_to_one and dst is not None and dst != group.ranks[group.rank]:      # dst is a global rank
        return
    out = tensor if tensor.is_contiguous() else torch.empty_like(total)
    _tree_merge(total, row_max, out, finish=True)
    if out is not tensor:
        tensor.copy_(out)


def add_collective(tensor: torch.Tensor, op, group: LocalGroup, dst: Optional[int] = None) -> None:
    """utils/attn_bwd_dsl.py:28-35 as it is meant (the reference assigns the sum to a local name): the SUM
    all-reduce of the gradient partials of all ranks of ``group``, written into ``tensor`` in place."""
    if not _is_collective(op, "all_reduce"):
        raise ValueError("not support other op than all reduce")
    total = None
    for p in group.operands(tensor):
        total = p.to(torch.float32, copy=True) if total is None else total.add_(p)
    tensor.copy_(total)


def pack_block(block_out: torch.Tensor, block_lse: torch.Tensor,
               reduce_into: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``torch.cat([block_out.float(), block_lse.transpose(-2,-1).unsqueeze(-1)], -1)``
    (utils/flash_attn_dsl.py:396) in one pass; with ``reduce_into`` the result is
    ``flash_reduce(reduce_into, pack)`` without materialising the pack."""
    N.require_cuda(block_out, block_lse, reduce_into)
    B, Sq, Hq, D = block_out.shape
    block_out, block_lse = block_out.contiguous(), block_lse.contiguous()
    if block_out.dtype != torch.bfloat16:
        raise RuntimeError("block_out must be bfloat16")
    dst = torch.empty((B, Sq, Hq, D + 1), dtype=torch.float32, device=block_out.device)
    lhs = None if reduce_into is None else reduce_into.contiguous()
    with torch.cuda.device(block_out.device):
        code = N.lib().mhip_pack_reduce(N.ptr(lhs), N.ptr(block_out), N.ptr(block_lse), N.ptr(dst),
                                        B, Sq, Hq, D, N.stream_of(block_out))
    N.check(code, "mhip_pack_reduce")
    return dst


def unpack_into(buf: torch.Tensor, out: torch.Tensor, lse: torch.Tensor) -> None:
    """``out[...] = buf[..., :-1].to(out.dtype)``, ``lse[...] = buf[..., -1].transpose(1, 2)`` (the stores after
    the managed reduction, utils/flash_attn_dsl.py:406-407) in one pass: buf (B,Sq,Hq,D+1) fp32, out
    (B,Sq,Hq,D) bf16 contiguous, lse (B,Hq,Sq) fp32 contiguous."""
    N.require_cuda(buf, out, lse)
    B, Sq, Hq, W = buf.shape
    D = W - 1
    if buf.dtype != torch.float32 or out.shape != (B, Sq, Hq, D) or lse.shape != (B, Hq, Sq):
        raise RuntimeError("unpack_into takes a float32 (B,Sq,Hq,D+1) buffer, out (B,Sq,Hq,D) and lse (B,Hq,Sq)")
    if out.dtype != torch.bfloat16 or lse.dtype != torch.float32 or not (out.is_contiguous() and lse.is_contiguous()):
        raise RuntimeError("out must be contiguous bfloat16 and lse contiguous float32")
    buf = buf.contiguous()
    with torch.cuda.device(buf.device):
        code = N.lib().mhip_unpack(N.ptr(buf), N.ptr(out), N.ptr(lse), B, Sq, Hq, D, N.stream_of(buf))
    N.check(code, "mhip_unpack")


def grad_accumulate(acc: Optional[torch.Tensor], block: torch.Tensor) -> torch.Tensor:
    """``torch.add(acc, block.to(torch.float32))`` (utils/attn_bwd_dsl.py:117-129); ``acc is None``
    is the first chunk (codegen.py:99-115 emits a plain assignment there)."""
    N.require_cuda(acc, block)
    if block.dtype != torch.bfloat16:
        raise RuntimeError("block must be bfloat16")
    block = block.contiguous()
    if block.data_ptr() % 16:                      # a contiguous view that starts in the middle of a 16-byte group
        block = block.clone()
    dst = torch.empty(block.shape, dtype=torch.float32, device=block.device)
    a = None if acc is None else acc.contiguous()
    if a is not None and a.data_ptr() % 16:
        a = a.clone()
    with torch.cuda.device(block.device):
        code = N.lib().mhip_grad_accumulate(N.ptr(a), N.ptr(block), N.ptr(dst), block.numel(), N.stream_of(block))
    N.check(code, "mhip_grad_accumulate")
    return dst
