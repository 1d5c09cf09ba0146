"""Block forward / backward operators with the keyword surface Mercury's generated ring code calls.

The reference imports ``_flash_attn_forward`` / ``_flash_attn_backward`` from the third-party
``flash_attn.flash_attn_interface`` (utils/flash_attn_dsl.py:6, utils/attn_bwd_dsl.py:8) and
calls them by keyword with a dict built by ``get_default_args`` (utils/flash_attn_dsl.py:14-29,
159-176; utils/attn_bwd_dsl.py:86-115).  The two operators below are registered through
``torch.library.custom_op`` -- so ``get_default_args`` finds the Python signature on
``._init_fn`` exactly as it does for flash-attn >= 2.7 -- and forward to the gfx950 kernels behind
the C ABI of include/mercury_hip.h.  Binding these names into the namespace the generated code is
``exec``-ed in replaces flash-attn without touching the generated code.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _native as N

__all__ = ["_flash_attn_forward", "_flash_attn_backward", "attn_fwd_block", "attn_bwd_block"]


def _strides3(t: torch.Tensor):
    return t.stride(0), t.stride(1), t.stride(2)


def _check_block_inputs(q, k, v, dropout_p, window_size_left, window_size_right, softcap, alibi_slopes, causal=False):
    N.require_cuda(q, k, v)
    if dropout_p not in (0, 0.0, None):
        raise RuntimeError("dropout_p != 0 is not supported (the ring templates always pass 0)")
    if softcap not in (0, 0.0, None):
        raise RuntimeError("softcap != 0 is not supported")
    if alibi_slopes is not None:
        raise RuntimeError("alibi_slopes is not supported")
    # a right window of 0 is how flash-attn spells the causal mask; without `causal` it would be a mask of its own
    if (window_size_left not in (-1, None)) or (window_size_right not in ((-1, 0, None) if causal else (-1, None))):
        raise RuntimeError("sliding windows are not supported (window_size must be (-1, -1), or (-1, 0) with causal=True)")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise RuntimeError("q, k, v must be (batch, seq, heads, head_dim)")
    if q.stride(-1) != 1 or k.stride(-1) != 1 or v.stride(-1) != 1:
        raise RuntimeError("q, k, v must have a contiguous last dimension")
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[3]:
        raise RuntimeError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if q.shape[2] % k.shape[2] != 0:
        raise RuntimeError("number of query heads must be a multiple of the number of KV heads")


_DESCALE_CONSTANTS = {}


def _descale_pointer(t, device):
    """A descale as the kernel wants it: one float32 in device memory, read by the kernel when it runs.  A tensor is
    passed as it is (no copy to the host, no synchronisation: a step that re-quantises its operands every time, or
    a captured graph whose scales are rewritten between replays, sees the current value); a Python number becomes
    a one-element device tensor, made once per (device, value) and kept."""
    if t is None:
        return None
    if isinstance(t, torch.Tensor):
        if t.numel() != 1 or t.dtype != torch.float32:
            raise RuntimeError("a descale must be a float32 tensor with one element (per-tensor scale)")
        return t
    key = (str(device), float(t))
    cached = _DESCALE_CONSTANTS.get(key)
    if cached is None:
        cached = torch.tensor([float(t)], dtype=torch.float32, device=device)
        _DESCALE_CONSTANTS[key] = cached
    return cached


def attn_fwd_block(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float,
                   causal: bool = False, q_descale: Optional[torch.Tensor] = None,
                   k_descale: Optional[torch.Tensor] = None, v_descale: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                   ) -> Tuple[torch.Tensor, torch.Tensor]:
    """(Q shard, one KV chunk) -> (out (B,Sq,Hq,D), lse (B,Hq,Sq) fp32) through mhip_attn_fwd_block.
    bfloat16: any head dimension that is a multiple of 8 up to 128 (the kernels work on 128 columns and fill the
    missing ones with zeros on chip, which changes neither the scores nor the columns that exist);
    float8_e4m3fn: any multiple of 16 up to 128, in the same way."""
    _check_block_inputs(q, k, v, 0, -1, -1, 0.0, None)
    N.require_cuda(out, lse)
    B, Sq, Hq, D = q.shape
    _, Sc, Hkv, _ = k.shape
    if q.dtype == torch.bfloat16:
        dt, out_dtype = N.MHIP_BF16, torch.bfloat16
    elif q.dtype == torch.float8_e4m3fn:
        dt, out_dtype = N.MHIP_E4M3, torch.bfloat16
    else:
        raise RuntimeError(f"unsupported dtype {q.dtype}: the gfx950 kernels take bfloat16 or float8_e4m3fn")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("q, k, v must share one dtype")
    if out is None:
        out = torch.empty((B, Sq, Hq, D), dtype=out_dtype, device=q.device)
    elif out.shape != (B, Sq, Hq, D) or out.dtype != out_dtype or out.stride(-1) != 1:
        raise RuntimeError("out must be (B, Sq, Hq, D) bfloat16 with a contiguous last dimension")
    if lse is None:
        lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    elif lse.shape != (B, Hq, Sq) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise RuntimeError("lse must be a contiguous float32 (B, Hq, Sq) tensor")
    ds = [_descale_pointer(t, q.device) for t in (q_descale, k_descale, v_descale)]
    N.require_cuda(*ds)
    with torch.cuda.device(q.device):
        code = N.lib().mhip_attn_fwd_block(
            N.ptr(q), N.ptr(k), N.ptr(v), N.ptr(out), N.ptr(lse),
            B, Sq, Sc, Hq, Hkv, D,
            *_strides3(q), *_strides3(k), *_strides3(v), *_strides3(out),
            float(softmax_scale), N.MASK_CAUSAL if causal else N.MASK_NONE, dt,
            N.ptr(ds[0]), N.ptr(ds[1]), N.ptr(ds[2]), N.stream_of(q))
    N.check(code, "mhip_attn_fwd_block")
    return out, lse


@torch.library.custom_op("mercury_amd::_flash_attn_forward", mutates_args=(), device_types="cuda")
def _flash_attn_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    dropout_p: float,
    softmax_scale: float,
    causal: bool,
    window_size_left: int,
    window_size_right: int,
    softcap: float,
    alibi_slopes: Optional[torch.Tensor],
    return_softmax: bool,
    q_descale: Optional[torch.Tensor] = None,
    k_descale: Optional[torch.Tensor] = None,
    v_descale: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(out, softmax_lse, S_dmask, rng_state)``; the last two are empty placeholders
    (no dropout), kept because the generated code asserts ``len(outputs) == 4``
    (utils/flash_attn_dsl.py:175)."""
    _check_block_inputs(q, k, v, dropout_p, window_size_left, window_size_right, softcap, alibi_slopes, causal)
    out, lse = attn_fwd_block(q, k, v, softmax_scale, bool(causal), q_descale, k_descale, v_descale)
    empty = torch.empty((0,), dtype=q.dtype if q.dtype == torch.bfloat16 else torch.bfloat16, device=q.device)
    rng = torch.empty((2,), dtype=torch.int64, device=q.device)
    return out, lse, empty, rng


@_flash_attn_forward.register_fake
def _(q, k, v, dropout_p, softmax_scale, causal, window_size_left, window_size_right, softcap,
      alibi_slopes, return_softmax, q_descale=None, k_descale=None, v_descale=None):
    B, Sq, Hq, D = q.shape
    od = torch.bfloat16
    return (q.new_empty((B, Sq, Hq, D), dtype=od), q.new_empty((B, Hq, Sq), dtype=torch.float32),
            q.new_empty((0,), dtype=od), q.new_empty((2,), dtype=torch.int64))


def attn_bwd_block(dout, q, k, v, out, softmax_lse, dq, dk, dv, softmax_scale, causal=False,
                   deterministic=False, dq_acc: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Block backward through mhip_attn_bwd_block; writes every element of dq, dk, dv in place and, if
    ``dq_acc`` (fp32, contiguous, q's shape) is given, also adds the block's dq into it.  Returns
    delta = rowsum(dout * out) as the kernel computed it, (B, Hq, Sq) fp32."""
    _check_block_inputs(q, k, v, 0, -1, -1, 0.0, None)
    N.require_cuda(dout, out, softmax_lse, dq, dk, dv, dq_acc)
    B, Sq, Hq, D = q.shape
    _, Sc, Hkv, _ = k.shape
    if q.dtype != torch.bfloat16:
        raise RuntimeError("the backward kernel takes bfloat16 only")
    for name, t, like in (("dout", dout, q), ("out", out, q), ("dq", dq, q), ("dk", dk, k), ("dv", dv, k)):
        if t.shape != like.shape or t.dtype != torch.bfloat16:
            raise RuntimeError(f"{name} must be bfloat16 with shape {tuple(like.shape)}")
    if softmax_lse.shape != (B, Hq, Sq) or softmax_lse.dtype != torch.float32:
        raise RuntimeError("softmax_lse must be float32 (B, Hq, Sq)")
    softmax_lse = softmax_lse.contiguous()
    if dq_acc is not None and (dq_acc.shape != q.shape or dq_acc.dtype != torch.float32
                               or not dq_acc.is_contiguous()):
        raise RuntimeError("dq_acc must be a contiguous float32 tensor of q's shape")

    # the C ABI takes one stride triple each for (q, dout), (k, v), (dk, dv), dq and out
    def same(*ts):
        return all(t.stride() == ts[0].stride() for t in ts)

    def rows_ok(t):
        return t.stride(-1) == 1 and all(st % 8 == 0 for st in t.stride()[:-1])
    qq, dd = (q, dout) if same(q, dout) and rows_ok(q) else (q.contiguous(), dout.contiguous())
    oo = out if rows_ok(out) else out.contiguous()
    dq_w = dq if rows_ok(dq) else torch.empty_like(q, memory_format=torch.contiguous_format)
    kk, vv = (k, v) if same(k, v) and rows_ok(k) else (k.contiguous(), v.contiguous())
    dk_w, dv_w = (dk, dv) if same(dk, dv) and rows_ok(dk) else \
        (torch.empty_like(k, memory_format=torch.contiguous_format),
         torch.empty_like(v, memory_format=torch.contiguous_format))
    lib = N.lib()
    ws = torch.empty((int(lib.mhip_attn_bwd_workspace_bytes(B, Sq, Sc, Hq, Hkv, D)),), dtype=torch.uint8,
                     device=q.device)
    with torch.cuda.device(q.device):
        code = lib.mhip_attn_bwd_block(
            N.ptr(dd), N.ptr(qq), N.ptr(kk), N.ptr(vv), N.ptr(oo), N.ptr(softmax_lse),
            N.ptr(dq_w), N.ptr(dk_w), N.ptr(dv_w), N.ptr(dq_acc),
            B, Sq, Sc, Hq, Hkv, D,
            *_strides3(qq), *_strides3(kk), *_strides3(dk_w), *_strides3(dq_w), *_strides3(oo),
            float(softmax_scale), N.MASK_CAUSAL if causal else N.MASK_NONE, int(bool(deterministic)),
            N.ptr(ws), N.stream_of(q))
    N.check(code, "mhip_attn_bwd_block")
    if dq_w is not dq:
        dq.copy_(dq_w)
    if dk_w is not dk:
        dk.copy_(dk_w)
        dv.copy_(dv_w)
    # the workspace is (-delta | lse in base 2 | delta), (B, Hq, Sq) fp32 each in a slot rounded up to 4 elements:
    # the last one is flash-attn's softmax_d, handed back as a view (no extra kernel, no extra allocation)
    rows = B * Hq * Sq
    slot = (rows + 3) & ~3
    return ws.view(torch.float32)[2 * slot: 2 * slot + rows].view(B, Hq, Sq)


@torch.library.custom_op("mercury_amd::_flash_attn_backward", mutates_args=("dq", "dk", "dv"),
                         device_types="cuda")
def _flash_attn_backward(
    dout: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    softmax_lse: torch.Tensor,
    dq: torch.Tensor,
    dk: torch.Tensor,
    dv: torch.Tensor,
    dropout_p: float,
    softmax_scale: float,
    causal: bool,
    window_size_left: int,
    window_size_right: int,
    softcap: float,
    alibi_slopes: Optional[torch.Tensor],
    deterministic: bool,
    rng_state: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Keyword surface of utils/attn_bwd_dsl.py:86-115; dq/dk/dv are caller-allocated
    (``torch.empty``, utils/attn_bwd_dsl.py:83-84) and every element of them is written.
    Returns ``softmax_d`` (rowsum(dout * out), (B,Hq,Sq) fp32) like flash-attn does."""
    _check_block_inputs(q, k, v, dropout_p, window_size_left, window_size_right, softcap, alibi_slopes, causal)
    return attn_bwd_block(dout, q, k, v, out, softmax_lse, dq, dk, dv, softmax_scale, bool(causal),
                          bool(deterministic))
