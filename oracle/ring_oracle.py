"""fp32/fp64 CPU restatement of the per-rank ring-attention step.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Every function cites the reference lines it restates (paths are relative to the
reference tree).  The block kernel itself lives in the third-party package
``flash-attn>=2.7.0`` (reference ``setup.py:16``), which is not vendored; its
published contract is restated here from the call sites
``utils/flash_attn_dsl.py:159-176`` and ``utils/attn_bwd_dsl.py:83-115``:

* forward:  ``out = softmax(scale * q k^T) v`` and
  ``lse = logsumexp(scale * q k^T, -1)`` (natural log), GQA by repeating each
  KV head ``Hq/Hkv`` times, causal mask aligned to the bottom-right corner
  (query ``i`` sees key ``j`` iff ``j <= i + Sk - Sq``), rows with no visible
  key give ``out = 0`` and ``lse = -inf``;
* backward: recompute ``P = exp(scale * q k^T - lse)`` from the saved LSE,
  ``delta = rowsum(dout * out)``, ``dV = P^T dout``, ``dP = dout v^T``,
  ``dS = P * (dP - delta)``, ``dQ = scale * dS k``, ``dK = scale * dS^T q``.

How each function is pinned (see tests/test_oracle_pins.py): brute-force loops
on tiny shapes, torch library routines (softmax, logsumexp, logaddexp,
scaled_dot_product_attention, autograd), closed forms of the merge, and a
message-passing simulation of the ring for the schedules.  The reference holds
no golden vector for this path, so none is used.
"""
from __future__ import annotations

import math
from typing import Iterable, List, Optional, Sequence, Tuple

import torch

__all__ = [
    "block_attention", "single_pass_attention", "merge_reference", "merge_closed_form",
    "update_out_and_lse", "merge_chain", "pack_block", "flash_reduce", "tree_merge", "block_backward",
    "single_ring_order", "double_ring_order", "ring_divide_order",
    "zigzag_blocks", "zigzag_step", "zigzag_local_positions",
    "quantize_e4m3", "dequantize", "e4m3_p_rounding_bound",
    "ring_forward", "ring_forward_packed", "ring_backward", "zigzag_ring_forward",
]

E4M3_MAX = 448.0


# --------------------------------------------------------------------------------------
# block forward  (contract of _flash_attn_forward at utils/flash_attn_dsl.py:159-176)
# --------------------------------------------------------------------------------------
def block_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float,
                    causal: bool = False, dtype: torch.dtype = torch.float32,
                    ) -> Tuple[torch.Tensor, torch.Tensor]:
    """One Q shard against one KV chunk.

    q ``(B,Sq,Hq,D)``, k/v ``(B,Sc,Hkv,D)`` -> out ``(B,Sq,Hq,D)``, lse ``(B,Hq,Sq)``,
    both in ``dtype``.  Loops over (batch, head) so the score matrix never exceeds
    ``Sq x Sc`` elements.
    """
    B, Sq, Hq, D = q.shape
    Bk, Sc, Hkv, Dk = k.shape
    assert (B, D) == (Bk, Dk) and v.shape == k.shape and Hq % Hkv == 0
    group = Hq // Hkv
    out = torch.zeros(B, Sq, Hq, D, dtype=dtype)
    lse = torch.full((B, Hq, Sq), -math.inf, dtype=dtype)
    if Sq == 0 or Sc == 0:
        return out, lse
    mask = None
    if causal:
        i = torch.arange(Sq).unsqueeze(1)
        j = torch.arange(Sc).unsqueeze(0)
        mask = j > i + (Sc - Sq)           # True = hidden
    for b in range(B):
        for h in range(Hq):
            qh = q[b, :, h, :].to(dtype)
            kh = k[b, :, h // group, :].to(dtype)
            vh = v[b, :, h // group, :].to(dtype)
            s = (qh @ kh.t()) * softmax_scale
            if mask is not None:
                s = s.masked_fill(mask, -math.inf)
            l = torch.logsumexp(s, dim=-1)
            p = torch.exp(s - torch.where(torch.isinf(l), torch.zeros_like(l), l).unsqueeze(-1))
            out[b, :, h, :] = p @ vh
            lse[b, h, :] = l
    return out, lse


def single_pass_attention(q, k, v, softmax_scale, causal=False, dtype=torch.float32):
    """Attention over the whole key sequence at once: what the reference's tests compare
    the ring result with (``flash_attn_qkvpacked_func`` at ``example.py:169``)."""
    return block_attention(q, k, v, softmax_scale, causal=causal, dtype=dtype)


# --------------------------------------------------------------------------------------
# merge  (utils/flash_attn_dsl.py:31-71, 293-305, 396)
# --------------------------------------------------------------------------------------
def merge_reference(out, lse, block_out, block_lse):
    """``_update_out_and_lse`` exactly as written at utils/flash_attn_dsl.py:38-47.

    out ``(B,Sq,Hq,D)``, lse ``(B,Sq,Hq,1)``, block_out ``(B,Sq,Hq,D)`` any dtype,
    block_lse ``(B,Hq,Sq)``.  NaNs when both LSEs are ``-inf`` or the accumulator's is
    (the reference does as well).
    """
    bo = block_out.to(out.dtype)
    bl = block_lse.transpose(-2, -1).unsqueeze(-1).to(lse.dtype)
    new_out = out - torch.sigmoid(bl - lse) * (out - bo)
    new_lse = lse - torch.nn.functional.logsigmoid(lse - bl)
    return new_out, new_lse


def merge_closed_form(out, lse, block_out, block_lse):
    """The closed form stated in the comment at utils/flash_attn_dsl.py:42-43:
    ``lse' = logaddexp(lse, bl)``, ``out' = e^{lse-lse'} out + e^{bl-lse'} bo``;
    ``-inf`` operands are the identity (limit of the reference's formula)."""
    bo = block_out.to(out.dtype)
    bl = block_lse.transpose(-2, -1).unsqueeze(-1).to(lse.dtype)
    new_lse = torch.logaddexp(lse, bl)
    safe = torch.where(torch.isinf(new_lse), torch.zeros_like(new_lse), new_lse)
    new_out = torch.exp(lse - safe) * out + torch.exp(bl - safe) * bo
    return new_out, new_lse


def update_out_and_lse(out, lse, block_out, block_lse, slice_=None, merge=merge_closed_form,
                       acc_dtype=torch.float32):
    """Dispatch of utils/flash_attn_dsl.py:51-71: first call initialises, ``slice_``
    merges a sub-range in place, otherwise a functional merge."""
    if out is None:
        if slice_ is not None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        out = block_out.to(acc_dtype)
        lse = block_lse.transpose(-2, -1).unsqueeze(-1).to(acc_dtype)
    elif slice_ is not None:
        so, sl = merge(out[slice_], lse[slice_], block_out, block_lse)
        out[slice_], lse[slice_] = so, sl
    else:
        out, lse = merge(out, lse, block_out, block_lse)
    return out, lse


def merge_chain(block_outs, block_lses, acc_dtype=torch.float64):
    """The chunk loop's chain of ``update_out_and_lse`` calls over all block results followed by the
    stores of utils/flash_attn_dsl.py:178-179: returns ``(out (B,Sq,Hq,D), lse (B,Hq,Sq))`` in
    ``acc_dtype``.  Built from the pinned pieces above; what a one-pass fold of all blocks has to equal."""
    out = lse = None
    for bo, bl in zip(block_outs, block_lses):
        out, lse = update_out_and_lse(out, lse, bo, bl, acc_dtype=acc_dtype)
    return out, lse.squeeze(dim=-1).transpose(1, 2)


def pack_block(block_out, block_lse):
    """utils/flash_attn_dsl.py:396 -- ``(B,Sq,Hq,D+1)`` fp32, LSE in the last column."""
    return torch.cat([block_out.to(torch.float32),
                      block_lse.transpose(-2, -1).unsqueeze(-1).to(torch.float32)], dim=-1)


def flash_reduce(lhs, rhs):
    """utils/flash_attn_dsl.py:293-305 on packed operands (closed form, -inf safe)."""
    l_out, l_lse = lhs[..., :-1], lhs[..., -1:]
    r_out, r_lse = rhs[..., :-1], rhs[..., -1:]
    lse = torch.logaddexp(l_lse, r_lse)
    safe = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)
    out = torch.exp(l_lse - safe) * l_out + torch.exp(r_lse - safe) * r_out
    return torch.cat([out, lse], dim=-1)


# --------------------------------------------------------------------------------------
# block backward  (contract of _flash_attn_backward at utils/attn_bwd_dsl.py:83-115)
# --------------------------------------------------------------------------------------
def tree_merge(packed_per_rank: Sequence[torch.Tensor]) -> torch.Tensor:
    """Tree-attention merge of the packed ``(out | lse)`` partial results of all ranks, as
    utils/flash_attn_dsl.py:307-324 does it with collectives: ``m = MAX lse``, ``d = exp(lse - m)``,
    ``out = SUM(out * d) / SUM(d)``, ``lse = m + log SUM(d)``.  Rows that are -inf on every rank give
    (0 | -inf) here (the reference would produce NaN).  Pinned in the tests against folding the same
    operands pairwise with the closed-form merge."""
    outs = [p[..., :-1].double() for p in packed_per_rank]
    lses = [p[..., -1:].double() for p in packed_per_rank]
    m = lses[0]
    for l in lses[1:]:
        m = torch.maximum(m, l)
    safe_m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    ds = [torch.exp(l - safe_m) for l in lses]
    sum_d = sum(ds)
    sum_out = sum(o * d for o, d in zip(outs, ds))
    out = torch.where(sum_d > 0, sum_out / sum_d.clamp_min(1e-300), torch.zeros_like(sum_out))
    lse = torch.where(sum_d > 0, m + torch.log(sum_d.clamp_min(1e-300)), torch.full_like(m, -math.inf))
    return torch.cat([out, lse], dim=-1).to(packed_per_rank[0].dtype)


def block_backward(dout, q, k, v, out, lse, softmax_scale, causal=False, dtype=torch.float32):
    """Gradients of one (Q shard, KV chunk) block given the *final merged* ``out`` and
    ``lse`` (utils/attn_bwd_dsl.py:73-76 loads them unchanged for every chunk).

    Returns dq ``(B,Sq,Hq,D)``, dk, dv ``(B,Sc,Hkv,D)`` in ``dtype``.
    """
    B, Sq, Hq, D = q.shape
    _, Sc, Hkv, _ = k.shape
    group = Hq // Hkv
    dq = torch.zeros(B, Sq, Hq, D, dtype=dtype)
    dk = torch.zeros(B, Sc, Hkv, D, dtype=dtype)
    dv = torch.zeros(B, Sc, Hkv, D, dtype=dtype)
    mask = None
    if causal:
        i = torch.arange(Sq).unsqueeze(1)
        j = torch.arange(Sc).unsqueeze(0)
        mask = j > i + (Sc - Sq)
    for b in range(B):
        for h in range(Hq):
            g = h // group
            qh, kh, vh = (t.to(dtype) for t in (q[b, :, h], k[b, :, g], v[b, :, g]))
            doh, oh = dout[b, :, h].to(dtype), out[b, :, h].to(dtype)
            l = lse[b, h].to(dtype)
            s = (qh @ kh.t()) * softmax_scale
            if mask is not None:
                s = s.masked_fill(mask, -math.inf)
            p = torch.exp(s - torch.where(torch.isinf(l), torch.zeros_like(l), l).unsqueeze(-1))
            if mask is not None:
                p = p.masked_fill(mask, 0.0)
            delta = (doh * oh).sum(-1, keepdim=True)
            dv[b, :, g] += p.t() @ doh
            dp = doh @ vh.t()
            ds = p * (dp - delta)
            dq[b, :, h] = softmax_scale * (ds @ kh)
            dk[b, :, g] += softmax_scale * (ds.t() @ qh)
    return dq, dk, dv


# --------------------------------------------------------------------------------------
# schedules  (mercury/backend/pytorch/codegen.py:292-314,443-494; backend/pytorch/utils.py:41-106)
# --------------------------------------------------------------------------------------
def single_ring_order(rank: int, world: int) -> List[int]:
    """Chunk held at ring step i: every rank sends to ``rank+1`` and receives from
    ``rank-1`` (codegen.py:480-491 with ``shift_tuple_element(indices, 0, +1/-1, W)``), and
    chunk id == source rank (``qkv.chunk(W, dim=1)[rank]``, example.py:161)."""
    return [(rank - i) % world for i in range(world)]


def double_ring_order(rank: int, inner: int, outer: int) -> List[int]:
    """Order for a ``(inner, outer)`` mesh (tests/test_double_ring.py:56,80,84): mesh dim 0
    is the fastest rank digit (utils.py:41-82), the generated loops are
    ``for outer: for inner:`` and a hop goes over dim 0 unless the inner loop is at its
    last step, then over dim 1 (codegen.py:480-491)."""
    a, b = rank % inner, rank // inner
    return [((b - o) % outer) * inner + ((a - i + o) % inner)
            for o in range(outer) for i in range(inner)]


def ring_divide_order(rank: int, world: int, divide: int) -> List[Tuple[int, int]]:
    """(chunk, sub-chunk) pairs when ``ring_divide = divide``: an outer loop over the
    sub-chunk wraps the ring loop (codegen.py:299-306)."""
    return [((rank - i) % world, s) for s in range(divide) for i in range(world)]


# --------------------------------------------------------------------------------------
# zigzag causal layout (not in the reference; only the slice_ hook at
# utils/flash_attn_dsl.py:56,63-68 exists).  Rank r of W holds blocks r and 2W-1-r of 2W.
# --------------------------------------------------------------------------------------
def zigzag_blocks(rank: int, world: int) -> Tuple[int, int]:
    return rank, 2 * world - 1 - rank


def zigzag_local_positions(rank: int, world: int, block: int) -> torch.Tensor:
    """Global token position of each local row (two blocks of ``block`` rows)."""
    lo, hi = zigzag_blocks(rank, world)
    return torch.cat([torch.arange(lo * block, (lo + 1) * block),
                      torch.arange(hi * block, (hi + 1) * block)])


def zigzag_step(rank: int, step: int, world: int) -> Tuple[str, int]:
    """Class of ring step ``step`` on ``rank``: ``("diag", src)`` -- causal over the local
    square; ``("kv_first_half", src)`` -- all Q rows against the first half of the chunk,
    no mask; ``("q_second_half", src)`` -- second half of the Q rows against the whole
    chunk, no mask, merged through ``slice_``."""
    src = (rank - step) % world
    if step == 0:
        return "diag", src
    return ("kv_first_half", src) if src < rank else ("q_second_half", src)


# --------------------------------------------------------------------------------------
# fp8 (not in the reference): per-tensor scale amax/448, round-to-nearest-even e4m3
# --------------------------------------------------------------------------------------
def quantize_e4m3(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    amax = x.abs().max().to(torch.float32) if x.numel() else torch.zeros((), dtype=torch.float32)
    # amax / 448 in fp64, rounded once to fp32: the same bits on the host and on the device
    scale = torch.where(amax > 0, (amax.double() / 448.0).float(), torch.ones_like(amax))
    xq = (x.to(torch.float32) / scale).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return xq, scale


def dequantize(xq: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    return xq.to(torch.float32) * scale


# --------------------------------------------------------------------------------------
# ring-step drivers: the loop the code generator emits (mercury/backend/pytorch/codegen.py:264-355,
# 443-523) with the send/recv replaced by indexing a list of chunks
def e4m3_p_rounding_bound(q, k, v, softmax_scale, causal=False):
    """Per-element bound on what rounding the softmax numerators P to e4m3 (three mantissa bits: relative
    error at most 2^-4 per value) can do to ``out = sum_i P_i v_i / sum_i P_i`` when the denominator keeps
    the unrounded values: ``|error| <= 2^-4 * sum_i w_i |v_i|`` with ``w`` the softmax weights, i.e. 2^-4
    times attention over ``|v|``.  Used by the tests as the tolerance of the fp8 kernel against attention on
    the de-quantised operands (few visible keys and large |v| make it larger than any fixed number)."""
    amp, _ = block_attention(q, k, v.abs(), softmax_scale, causal=causal)
    return amp * 2.0 ** -4


# --------------------------------------------------------------------------------------
def ring_forward(q, kv_chunks: Sequence[torch.Tensor], order: Iterable[int], softmax_scale,
                 causal=False, dtype=torch.float32, block_out_dtype: Optional[torch.dtype] = None,
                 merge=merge_closed_form):
    """``kv_chunks[c]`` is ``(2,B,Sc,Hkv,D)``; returns out ``(B,Sq,Hq,D)`` and lse
    ``(B,Hq,Sq)`` in ``dtype`` (the epilogue of utils/flash_attn_dsl.py:178-179 without the
    cast to the input dtype).  ``block_out_dtype`` rounds each block result the way a bf16
    kernel output would before the merge upcasts it again."""
    out = lse = None
    for c in order:
        kv = kv_chunks[c]
        bo, bl = block_attention(q, kv[0], kv[1], softmax_scale, causal=causal, dtype=dtype)
        if block_out_dtype is not None:
            bo = bo.to(block_out_dtype)
        if out is None:
            out, lse = bo.to(dtype), bl.transpose(-2, -1).unsqueeze(-1).to(dtype)
        else:
            out, lse = merge(out, lse, bo, bl)
    return out, lse.squeeze(-1).transpose(1, 2).contiguous()


def ring_forward_packed(q, kv_chunks, order, softmax_scale, dtype=torch.float32):
    """The managed-reduction template (utils/flash_attn_dsl.py:370-408): pack every block
    result and fold with ``flash_reduce``; the first block initialises the buffer
    (codegen.py:99-115)."""
    buf = None
    for c in order:
        kv = kv_chunks[c]
        bo, bl = block_attention(q, kv[0], kv[1], softmax_scale, dtype=dtype)
        res = pack_block(bo, bl).to(dtype)
        buf = res if buf is None else flash_reduce(buf, res)
    return buf[..., :-1], buf[..., -1].transpose(1, 2).contiguous()


def ring_backward(q, kv_chunks, order, out, lse, dout, softmax_scale, dtype=torch.float32):
    """utils/attn_bwd_dsl.py:70-134: dq accumulates over chunks; each chunk's dk/dv is its own
    (one Q shard per rank, so the sum over ``s_q`` has one term here).  Returns dq and a dict
    chunk -> (dk, dv)."""
    dq = None
    dkv = {}
    for c in order:
        kv = kv_chunks[c]
        bdq, bdk, bdv = block_backward(dout, q, kv[0], kv[1], out, lse, softmax_scale, dtype=dtype)
        dq = bdq if dq is None else dq + bdq
        dkv[c] = (bdk, bdv)
    return dq, dkv


def zigzag_ring_forward(q, kv_chunks, rank, world, softmax_scale, dtype=torch.float32):
    """Causal ring step in the zigzag layout; ``q`` and every ``kv_chunks[c]`` hold the two
    blocks of their rank back to back along the sequence dimension."""
    Sq = q.shape[1]
    half = Sq // 2
    out = lse = None
    for step in range(world):
        kind, src = zigzag_step(rank, step, world)
        kv = kv_chunks[src]
        if kind == "diag":
            bo, bl = block_attention(q, kv[0], kv[1], softmax_scale, causal=True, dtype=dtype)
            out, lse = update_out_and_lse(out, lse, bo, bl, acc_dtype=dtype)
        elif kind == "kv_first_half":
            bo, bl = block_attention(q, kv[0][:, :half], kv[1][:, :half], softmax_scale, dtype=dtype)
            out, lse = update_out_and_lse(out, lse, bo, bl)
        else:
            bo, bl = block_attention(q[:, half:], kv[0], kv[1], softmax_scale, dtype=dtype)
            out, lse = update_out_and_lse(out, lse, bo, bl,
                                          slice_=(slice(None), slice(half, None)))
    return out, lse.squeeze(-1).transpose(1, 2).contiguous()
