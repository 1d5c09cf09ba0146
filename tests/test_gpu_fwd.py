"""Block forward kernel (through the C ABI) against the CPU oracle on the same seeded inputs.

Tolerances (bf16 inputs, fp32 oracle on the very same bf16 values):
  max-abs(out) <= 2e-2 and LSE relative error <= 1e-3   -- the stated bar for bf16;
  rel-L2(out)  <= 1e-2                                  -- own, tighter gate (N(0,1) data gives
                                                            |out| ~ 0.1, so max-abs alone is weak).
"""
import math

import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

OUT_ATOL = 2e-2
LSE_RTOL = 1e-3
REL_L2 = 1e-2


def _mk(B, Sq, Sc, Hq, Hkv, D=128, seed=0, qscale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Sq, Hq, D, generator=g) * qscale).bfloat16()
    kv = torch.randn(2, B, Sc, Hkv, D, generator=g).bfloat16()
    return q, kv


def _check(out, lse, ro, rl, tag=""):
    out, lse = out.float().cpu(), lse.float().cpu()
    assert not torch.isnan(out).any(), tag
    inf_ref = torch.isinf(rl)
    assert torch.equal(torch.isinf(lse), inf_ref), tag
    assert (out - ro).abs().max().item() <= OUT_ATOL, (tag, (out - ro).abs().max().item())
    denom = ro.norm().item()
    if denom > 0:
        assert (out - ro).norm().item() / denom <= REL_L2, (tag, (out - ro).norm().item() / denom)
    fin = ~inf_ref
    if fin.any():
        rel = ((lse[fin] - rl[fin]).abs() / rl[fin].abs().clamp_min(1.0)).max().item()
        assert rel <= LSE_RTOL, (tag, rel)


SHAPES = [
    # B, Sq, Sc, Hq, Hkv, causal
    (1, 128, 64, 1, 1, False),
    (1, 128, 128, 2, 2, False),
    (2, 256, 192, 4, 2, False),
    (1, 100, 77, 2, 1, False),      # ragged rows and keys
    (1, 1, 1, 1, 1, False),
    (1, 300, 130, 3, 3, False),
    (1, 512, 1024, 8, 2, False),    # GQA, several key tiles
    (1, 256, 256, 2, 2, True),
    (1, 200, 200, 2, 1, True),      # causal, ragged
    (1, 128, 320, 2, 2, True),      # causal with more keys than rows (bottom-right aligned)
    (1, 320, 128, 2, 2, True),      # causal with fewer keys: the first 192 rows see nothing
    (2, 130, 0, 2, 2, False),       # empty chunk
    (1, 384, 1100, 2, 1, False),    # 18 tiles, ragged: the four-stage LDS ring wraps several times
    (1, 384, 1100, 2, 1, True),
    (1, 257, 63, 1, 1, False),      # one ragged tile, a second workgroup with a single row
    (2, 600, 600, 8, 4, True),      # causal with B*Hq a multiple of 8: the per-XCD longest-first order
]


@pytest.mark.parametrize("B,Sq,Sc,Hq,Hkv,causal", SHAPES)
def test_fwd_block_matches_oracle(B, Sq, Sc, Hq, Hkv, causal):
    import mercury_artifact_amd as M

    print(f"case B{B} Sq{Sq} Sc{Sc} Hq{Hq} Hkv{Hkv} causal={causal}", flush=True)
    q, kv = _mk(B, Sq, Sc, Hq, Hkv)
    scale = 128 ** -0.5
    ro, rl = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale, causal=causal)
    qd, kvd = q.cuda(), kv.cuda()
    out, lse, s_dmask, rng = M._flash_attn_forward(
        q=qd, k=kvd[0], v=kvd[1], dropout_p=0, softmax_scale=scale, causal=causal,
        window_size_left=-1, window_size_right=-1, softcap=0.0, alibi_slopes=None, return_softmax=False)
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and out.shape == q.shape
    assert lse.dtype == torch.float32 and lse.shape == (B, Hq, Sq)
    _check(out, lse, ro, rl, "fwd")
    if Sc == 0:
        assert out.float().abs().max().item() == 0


def test_fwd_block_peaked_logits():
    """Large-magnitude scores: softmax concentrates on a few keys, errors in the max / rescale path
    would show as O(1) differences."""
    import mercury_artifact_amd as M

    q, kv = _mk(1, 256, 384, 4, 4, seed=3, qscale=6.0)
    scale = 128 ** -0.5
    ro, rl = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale)
    out, lse = M.attn_fwd_block(q.cuda(), kv[0].cuda(), kv[1].cuda(), scale)
    _check(out, lse, ro, rl, "peaked")


@pytest.mark.parametrize("direction", ["rising", "falling"])
@pytest.mark.parametrize("fp8", [False, True])
def test_fwd_block_monotone_scores(direction, fp8):
    """Scores that rise (or fall) by about 20 binades from one key tile to the next: with rising scores the
    reference the exponentials are taken against has to move on every tile and everything accumulated so far is
    rescaled by 2^-20 each time; with falling scores it must never move and later tiles underflow to nothing.
    The first 16 head-dim values carry the ramp, the rest is noise."""
    import mercury_artifact_amd as M

    B, Sq, Sc, H, D = 1, 96, 640, 2, 128
    g = torch.Generator().manual_seed(7)
    q = torch.randn(B, Sq, H, D, generator=g) * 0.25
    k = torch.randn(B, Sc, H, D, generator=g) * 0.25
    v = torch.randn(B, Sc, H, D, generator=g)
    ramp = torch.arange(Sc, dtype=torch.float32) / 64.0              # one unit per 64-key tile
    if direction == "falling":
        ramp = ramp.flip(0)
    q[..., :16] = 2.0
    k[..., :16] = (ramp * 5.0)[None, :, None, None] / 2.0            # q.k ramp = 16 * 2 * 2.5 * t = 80 t
    scale = D ** -0.5                                                # 80 * 0.088 * log2(e) = 10 binades per unit
    k[..., :16] *= 2.0                                               # -> 20 binades per tile
    if fp8:
        (qq, sq), (kq, sk), (vq, sv) = M.quantize_e4m3(q.cuda()), M.quantize_e4m3(k.cuda()), M.quantize_e4m3(v.cuda())
        ref_q, ref_k, ref_v = (O.dequantize(t.cpu(), s_.cpu()) for t, s_ in ((qq, sq), (kq, sk), (vq, sv)))
        ro, rl = O.block_attention(ref_q, ref_k, ref_v, scale)
        out, lse = M.attn_fwd_block(qq, kq, vq, scale, q_descale=sq, k_descale=sk, v_descale=sv)
        tol = 6e-2
    else:
        qb, kb, vb = q.bfloat16(), k.bfloat16(), v.bfloat16()
        ro, rl = O.block_attention(qb.float(), kb.float(), vb.float(), scale)
        out, lse = M.attn_fwd_block(qb.cuda(), kb.cuda(), vb.cuda(), scale)
        tol = 2e-2
    out, lse = out.float().cpu(), lse.cpu()
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert (out - ro).abs().max().item() <= tol
    assert ((lse - rl).abs() / rl.abs().clamp_min(1.0)).max().item() <= 1e-3


@pytest.mark.parametrize("direction", ["rising", "falling"])
@pytest.mark.parametrize("D", [128, 64, 40])
@pytest.mark.parametrize("causal", [False, True])
def test_fwd_block_monotone_scores_by_head_dim(direction, D, causal):
    """The same ramp of about 20 binades per key tile on the 64-column instantiation (D = 64: other slot
    arithmetic for the exponential pairs that ride in the matrix phase, the packed P overwritten right behind two
    O^T MFMAs) and on a head dimension below 128 of the 128-column one (D = 40), with and without the causal
    mask, so that the path that moves the reference runs together with masking.  The first 16 head-dim values
    carry the ramp."""
    import mercury_artifact_amd as M

    B, Sq, Sc, H = 1, 320, 640, 2
    g = torch.Generator().manual_seed(70 + D)
    q = torch.randn(B, Sq, H, D, generator=g) * 0.25
    k = torch.randn(B, Sc, H, D, generator=g) * 0.25
    v = torch.randn(B, Sc, H, D, generator=g)
    ramp = torch.arange(Sc, dtype=torch.float32) / 64.0
    if direction == "falling":
        ramp = ramp.flip(0)
    scale = D ** -0.5
    per_unit = 20.0 / (scale * 1.4426950408889634)                   # q.k increment that is 20 binades after scaling
    q[..., :16] = 2.0
    k[..., :16] = (ramp * per_unit / 32.0)[None, :, None, None]      # 16 columns x 2.0 x value
    qb, kb, vb = q.bfloat16(), k.bfloat16(), v.bfloat16()
    ro, rl = O.block_attention(qb.float(), kb.float(), vb.float(), scale, causal=causal)
    out, lse = M.attn_fwd_block(qb.cuda(), kb.cuda(), vb.cuda(), scale, causal=causal)
    out, lse = out.float().cpu(), lse.cpu()
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert (out - ro).abs().max().item() <= 2e-2
    assert ((lse - rl).abs() / rl.abs().clamp_min(1.0)).max().item() <= 1e-3


def test_fwd_block_strided_views_and_guard_bands():
    """k / v as halves of one packed tensor (storage offset != 0 for v), q as a row slice of a larger
    tensor, out written into the middle of a sentinel-filled buffer."""
    import mercury_artifact_amd as M

    B, Sq, Sc, H, D = 2, 192, 160, 2, 128
    g = torch.Generator().manual_seed(5)
    qbig = torch.randn(B, 2 * Sq, H, D, generator=g).bfloat16()
    kv = torch.randn(2, B, Sc, H, D, generator=g).bfloat16()
    q = qbig[:, Sq:]
    scale = 0.11
    ro, rl = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale)
    qd = qbig.cuda()[:, Sq:]
    kvd = kv.cuda()
    pad = 64
    obuf = torch.full((B, Sq + 2 * pad, H, D), 7.0, dtype=torch.bfloat16, device="cuda")
    lbuf = torch.full((B * H * Sq + 2 * pad,), 7.0, dtype=torch.float32, device="cuda")
    out_view = obuf[:, pad:pad + Sq]
    lse_view = lbuf[pad:pad + B * H * Sq].view(B, H, Sq)
    M.attn_fwd_block(qd, kvd[0], kvd[1], scale, out=out_view, lse=lse_view)
    torch.cuda.synchronize()
    _check(out_view, lse_view, ro, rl, "strided")
    assert (obuf[:, :pad] == 7.0).all() and (obuf[:, pad + Sq:] == 7.0).all()
    assert (lbuf[:pad] == 7.0).all() and (lbuf[-pad:] == 7.0).all()


@pytest.mark.parametrize("D", [64, 40])
def test_fwd_block_small_head_dim_reads_and_writes_only_its_columns(D):
    """q, k, v and out as COLUMN slices of 128-wide tensors whose other columns hold NaN (inputs) or a sentinel
    (output): a kernel that fetched or stored its full 128 on-chip columns would pick up the NaN or clobber the
    sentinel.  The slices keep the 128-element head stride, so nothing is copied on the way in."""
    import mercury_artifact_amd as M

    B, Sq, Sc, Hq, Hkv = 1, 200, 330, 4, 2
    q, kv = _mk(B, Sq, Sc, Hq, Hkv, D=D, seed=33)
    scale = D ** -0.5
    ro, rl = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale, causal=True)
    qw = torch.full((B, Sq, Hq, 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    kvw = torch.full((2, B, Sc, Hkv, 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    ow = torch.full((B, Sq, Hq, 128), 7.0, dtype=torch.bfloat16, device="cuda")
    for off in (0, 128 - D):                                    # the slice at the left and at the right edge
        qw.fill_(float("nan")); kvw.fill_(float("nan")); ow.fill_(7.0)
        qv, kvv, ov = qw[..., off:off + D], kvw[..., off:off + D], ow[..., off:off + D]
        qv.copy_(q.cuda()); kvv.copy_(kv.cuda())
        out, lse = M.attn_fwd_block(qv, kvv[0], kvv[1], scale, causal=True, out=ov)
        torch.cuda.synchronize()
        assert out is ov
        _check(ov, lse, ro, rl, f"D{D} off{off}")
        rest = torch.ones(128, dtype=torch.bool)
        rest[off:off + D] = False
        assert (ow[..., rest.cuda()] == 7.0).all()


def test_fwd_rejects_what_it_does_not_implement():
    import mercury_artifact_amd as M

    q, kv = _mk(1, 64, 64, 2, 2)
    qd, kvd = q.cuda(), kv.cuda()
    with pytest.raises(RuntimeError):
        M._flash_attn_forward(q=qd, k=kvd[0], v=kvd[1], dropout_p=0.1, softmax_scale=0.1, causal=False,
                              window_size_left=-1, window_size_right=-1, softcap=0.0, alibi_slopes=None,
                              return_softmax=False)
    with pytest.raises(RuntimeError):
        M.attn_fwd_block(qd[..., :100].contiguous(), kvd[0][..., :100].contiguous(),
                         kvd[1][..., :100].contiguous(), 0.1)     # head dim 100: not a multiple of 8
    big = torch.zeros(1, 64, 2, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError):
        M.attn_fwd_block(big, big, big, 0.1)                      # head dim 256: beyond the kernels' 128
    with pytest.raises(RuntimeError):
        M.attn_fwd_block(qd.float(), kvd[0].float(), kvd[1].float(), 0.1)
    with pytest.raises(RuntimeError):
        M.attn_fwd_block(q, kv[0], kv[1], 0.1)                    # CPU tensors: no fallback


def test_fwd_chunks_merge_to_single_pass_full_size():
    """The headline configuration (B1 H32 D128, Q 4096 x 8 chunks of 4096) at full size, checked through size-independent properties: the 8 merged
    chunk results equal one pass over all 32768 keys done by the same kernel (merge identity), and
    three heads are compared with the fp32 oracle."""
    import mercury_artifact_amd as M

    B, Sq, H, D, W = 1, 4096, 32, 128, 8
    torch.manual_seed(0)
    q = torch.randn(B, Sq, H, D).bfloat16()
    k = torch.randn(B, W * Sq, H, D).bfloat16()
    v = torch.randn(B, W * Sq, H, D).bfloat16()
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    chunks = [torch.stack([kd[:, c * Sq:(c + 1) * Sq], vd[:, c * Sq:(c + 1) * Sq]]) for c in range(W)]
    rank = 3
    ring = M.LocalRing((W,), rank, chunks)
    o = torch.empty_like(qd)
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    M.flash_attn_pack_kv(qd, chunks[rank], o, lse, scale, ring=ring)
    one_o, one_l = M.attn_fwd_block(qd, kd, vd, scale)
    torch.cuda.synchronize()
    assert (o.float() - one_o.float()).abs().max().item() <= 4e-3
    assert ((lse - one_l).abs() / one_l.abs()).max().item() <= 1e-5
    heads = [0, 13, 31]
    ro, rl = O.block_attention(q[:, :, heads].float(), k[:, :, heads].float(), v[:, :, heads].float(), scale)
    _check(o[:, :, heads], lse[:, heads], ro, rl, "config1")
    # every head on one window of 256 rows (rows 1792 .. 2047, across a workgroup boundary of the kernel)
    rows = slice(1792, 2048)
    ro, rl = O.block_attention(q[:, rows].float(), k.float(), v.float(), scale)
    _check(o[:, rows], lse[:, :, rows], ro, rl, "config1, all heads")


@pytest.mark.parametrize("D,causal", [(64, False), (64, True), (32, False), (96, True), (8, False), (120, True)])
def test_fwd_block_smaller_head_dims(D, causal):
    """Head dimensions below 128 (multiples of 8) run through the same kernel: the columns that do not exist are
    zeros on chip only (no padded copies)."""
    import mercury_artifact_amd as M

    B, Sq, Sc, Hq, Hkv = 2, 200, 330, 4, 2
    q, kv = _mk(B, Sq, Sc, Hq, Hkv, D=D, seed=31)
    scale = D ** -0.5
    ro, rl = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale, causal=causal)
    out, lse = M.attn_fwd_block(q.cuda(), kv[0].cuda(), kv[1].cuda(), scale, causal=causal)
    assert out.shape == (B, Sq, Hq, D) and out.is_contiguous()
    _check(out, lse, ro, rl, f"D{D}")
    into = torch.full((B, Sq, Hq, D), 7.0, dtype=torch.bfloat16, device="cuda")
    o2, l2 = M.attn_fwd_block(q.cuda(), kv[0].cuda(), kv[1].cuda(), scale, causal=causal, out=into)
    assert o2 is into and torch.equal(into, out) and torch.equal(l2, lse)


def test_config0_through_the_gpu_path():
    """The smallest benchmark configuration (the CPU plumbing case: B1 H4 D64, Q 1024 x 4 KV chunks of 256, N(0,1) from
    torch.manual_seed(0), scale 1/8) through libmercury_hip.so: the inputs are rounded to bf16 (the block
    operator takes no fp32, like the flash-attn operator it replaces) and every rank's ring step -- one fold,
    the literal chain, and unchanged generated-style text in the lazy namespace -- is compared with single-pass
    fp32 attention over all 1024 keys on the same rounded values."""
    import mercury_artifact_amd as M

    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 1024, 4, 64).bfloat16() for _ in range(3))
    scale = 64 ** -0.5
    chunks = [torch.stack([k[:, c * 256:(c + 1) * 256], v[:, c * 256:(c + 1) * 256]]) for c in range(4)]
    ref_o, ref_l = O.single_pass_attention(q.float(), k.float(), v.float(), scale)
    dev = [c.cuda() for c in chunks]
    qd = q.cuda()
    for rank in range(4):
        for deferred in (True, False):
            o = torch.empty_like(qd)
            lse = torch.empty(1, 4, 1024, dtype=torch.float32, device="cuda")
            M.flash_attn_pack_kv(qd, dev[rank], o, lse, scale, ring=M.LocalRing((4,), rank, dev),
                                 deferred_merge=deferred, fused_epilogue=deferred)
            _check(o, lse, ref_o, ref_l, f"config0 rank {rank} deferred={deferred}")


def test_block_operators_refuse_what_the_kernels_do_not_implement():
    """flash-attn arguments the ring templates never set (utils/flash_attn_dsl.py:159-173 passes dropout 0, no alibi,
    the window it was given, softcap 0): anything else is an error here, never a silently different result.  A right
    window of 0 is flash-attn's spelling of the causal mask and is accepted only together with ``causal``."""
    import mercury_artifact_amd as M

    B, S, H, D = 1, 64, 1, 128
    q = torch.randn(B, S, H, D, device="cuda").bfloat16()
    k, v = torch.randn_like(q), torch.randn_like(q)
    base = dict(q=q, k=k, v=v, dropout_p=0.0, softmax_scale=D ** -0.5, causal=False, window_size_left=-1,
                window_size_right=-1, softcap=0.0, alibi_slopes=None, return_softmax=False)
    M._flash_attn_forward(**base)
    M._flash_attn_forward(**dict(base, causal=True, window_size_right=0))
    for change in (dict(window_size_right=0), dict(window_size_left=16), dict(window_size_right=8, causal=True),
                   dict(dropout_p=0.1), dict(softcap=30.0), dict(alibi_slopes=torch.ones(H, device="cuda"))):
        with pytest.raises(RuntimeError, match="not supported"):
            M._flash_attn_forward(**dict(base, **change))
    out, lse = M.attn_fwd_block(q, k, v, D ** -0.5)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    back = dict(dout=q, q=q, k=k, v=v, out=out, softmax_lse=lse, dq=dq, dk=dk, dv=dv, dropout_p=0.0,
                softmax_scale=D ** -0.5, causal=False, window_size_left=-1, window_size_right=-1, softcap=0.0,
                alibi_slopes=None, deterministic=False, rng_state=None)
    M._flash_attn_backward(**back)
    for change in (dict(window_size_right=0), dict(window_size_left=16), dict(dropout_p=0.1), dict(softcap=30.0)):
        with pytest.raises(RuntimeError, match="not supported"):
            M._flash_attn_backward(**dict(back, **change))
