"""Block backward kernels (through the C ABI) against the CPU oracle on the same seeded inputs.

Tolerance: gradients come out in bf16 and P / dS are rounded to bf16 before the second contraction, so
each gradient is compared by relative L2 error <= 1.5e-2 and max-abs error <= 4e-2 * max|ref| against the
fp32 oracle on the same bf16 inputs.  The reference's own criterion (tests/test_attn_bwd.py:70-80,267-270:
inputs scaled by 1/100, mean |d| < 1e-3) is asserted as well."""
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return ((a - b).norm() / b.norm().clamp_min(1e-20)).item()


def _check_grad(name, got, ref):
    got = got.float().cpu()
    assert not torch.isnan(got).any(), name
    assert _rel(got, ref) <= 1.5e-2, (name, _rel(got, ref))
    assert (got - ref).abs().max().item() <= 4e-2 * ref.abs().max().item() + 1e-6, name


def _case(B, Sq, Sc, Hq, Hkv, causal, seed=0, in_scale=1.0, D=128):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Sq, Hq, D, generator=g) * in_scale).bfloat16()
    kv = (torch.randn(2, B, Sc, Hkv, D, generator=g) * in_scale).bfloat16()
    dout = (torch.randn(B, Sq, Hq, D, generator=g) * in_scale).bfloat16()
    scale = D ** -0.5
    o, lse = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale, causal=causal)
    o16 = o.bfloat16()
    rdq, rdk, rdv = O.block_backward(dout.float(), q.float(), kv[0].float(), kv[1].float(), o16.float(), lse,
                                     scale, causal=causal)
    return q, kv, dout, o16, lse, scale, (rdq, rdk, rdv)


BWD_SHAPES = [
    (1, 128, 128, 1, 1, False),
    (1, 256, 192, 2, 2, False),
    (2, 100, 77, 2, 1, False),       # ragged rows / keys, GQA
    (1, 300, 520, 4, 2, False),
    (1, 256, 256, 2, 2, True),
    (1, 200, 330, 2, 1, True),       # causal, bottom-right aligned, ragged
    (1, 330, 200, 2, 2, True),       # causal with rows that see no key
    (1, 640, 640, 2, 1, True),       # causal GQA, ten streamed tiles per head: the LDS ring wraps twice
    (1, 64, 700, 1, 1, False),       # few rows, many keys
    (1, 700, 64, 3, 1, False),       # many rows of three grouped heads, few keys
    (1, 1, 2, 1, 1, False),          # a single query row (with one key every gradient of q is exactly zero)
    (2, 384, 384, 8, 4, True),       # causal with B*Hq and B*Hkv multiples of 8: the per-XCD longest-first order
    (1, 1100, 900, 2, 2, False),     # five 256-row workgroups of the dQ pass, the last one ragged; 15 key tiles
    (1, 900, 1100, 2, 1, True),      # the same under the causal mask with more keys than rows, grouped heads
]


@pytest.mark.parametrize("B,Sq,Sc,Hq,Hkv,causal", BWD_SHAPES)
def test_bwd_block_matches_oracle(B, Sq, Sc, Hq, Hkv, causal):
    import mercury_artifact_amd as M

    print(f"bwd case B{B} Sq{Sq} Sc{Sc} Hq{Hq} Hkv{Hkv} causal={causal}", flush=True)
    q, kv, dout, o16, lse, scale, (rdq, rdk, rdv) = _case(B, Sq, Sc, Hq, Hkv, causal)
    qd, kvd, dd, od, ld = q.cuda(), kv.cuda(), dout.cuda(), o16.cuda(), lse.cuda()
    nan = float("nan")
    dq = torch.full_like(qd, nan)                     # the caller allocates with torch.empty: every
    dkv = torch.full_like(kvd, nan)                   # element must be overwritten
    ret = M._flash_attn_backward(
        dout=dd, q=qd, k=kvd[0], v=kvd[1], out=od, softmax_lse=ld, dq=dq, dk=dkv[0], dv=dkv[1],
        dropout_p=0, softmax_scale=scale, causal=causal, window_size_left=-1, window_size_right=-1,
        softcap=0.0, alibi_slopes=None, deterministic=False, rng_state=None)
    torch.cuda.synchronize()
    _check_grad("dq", dq, rdq)
    _check_grad("dk", dkv[0], rdk)
    _check_grad("dv", dkv[1], rdv)
    delta = (dout.float() * o16.float()).sum(-1).transpose(1, 2)
    assert torch.allclose(ret.cpu(), delta, atol=1e-3, rtol=1e-3)
    assert torch.equal(qd.cpu(), q) and torch.equal(kvd.cpu(), kv)      # inputs untouched


def test_bwd_reference_criterion_small_inputs():
    """tests/test_attn_bwd.py:70-80,267-270 of the reference: inputs / 100, mean |diff| < 1e-3."""
    import mercury_artifact_amd as M

    q, kv, dout, o16, lse, scale, (rdq, rdk, rdv) = _case(2, 512, 512, 4, 4, False, seed=1, in_scale=0.01)
    dq = torch.empty_like(q, device="cuda")
    dkv = torch.empty_like(kv, device="cuda")
    M.attn_bwd_block(dout.cuda(), q.cuda(), kv.cuda()[0], kv.cuda()[1], o16.cuda(), lse.cuda(),
                     dq, dkv[0], dkv[1], scale)
    assert (dq.float().cpu() - rdq).abs().mean().item() < 1e-3
    assert (dkv[0].float().cpu() - rdk).abs().mean().item() < 1e-3
    assert (dkv[1].float().cpu() - rdv).abs().mean().item() < 1e-3


def test_bwd_dq_accumulator_and_determinism():
    import mercury_artifact_amd as M

    q, kv, dout, o16, lse, scale, (rdq, _, _) = _case(1, 256, 256, 2, 2, False, seed=2)
    args = [t.cuda() for t in (dout, q, kv[0], kv[1], o16, lse)]
    runs = []
    acc = torch.zeros(q.shape, dtype=torch.float32, device="cuda")
    for _ in range(2):
        dq = torch.empty_like(args[1]); dk = torch.empty_like(args[2]); dv = torch.empty_like(args[3])
        M.attn_bwd_block(*args, dq, dk, dv, scale, dq_acc=acc)
        runs.append((dq.clone(), dk.clone(), dv.clone()))
    for a, b in zip(*runs):
        assert torch.equal(a, b)                       # no atomics: bitwise repeatable
    assert _rel(acc.cpu(), 2 * rdq) <= 5e-3             # fp32 accumulation of two identical blocks


@pytest.mark.parametrize("fused", [False, True])
def test_bwd_ring_step(fused):
    """The backward ring step (utils/attn_bwd_dsl.py:70-134 after `shift`): dq accumulates over the chunks,
    each chunk's dk/dv is compared with the oracle's."""
    import mercury_artifact_amd as M

    B, S, H, D, W, rank = 1, 1024, 3, 128, 4, 2
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, S // W, H, D, generator=g).bfloat16()
    kvs = [torch.randn(2, B, S // W, H, D, generator=g).bfloat16() for _ in range(W)]
    dout = torch.randn(B, S // W, H, D, generator=g).bfloat16()
    scale = D ** -0.5
    order = O.single_ring_order(rank, W)
    o, lse = O.ring_forward(q.float(), [c.float() for c in kvs], order, scale)
    o16 = o.bfloat16()
    rdq, rdkv = O.ring_backward(q.float(), [c.float() for c in kvs], order, o16.float(), lse, dout.float(), scale)
    dev = [c.cuda() for c in kvs]
    dq = torch.empty_like(q, device="cuda")
    dkv = torch.empty_like(dev[rank])
    got = {}
    M.flash_attn_backward(q.cuda(), dev[rank], o16.cuda(), lse.cuda(), dout.cuda(), dq, dkv, scale,
                          ring=M.LocalRing((W,), rank, dev), dkv_chunks=got, fused_accumulate=fused)
    torch.cuda.synchronize()
    _check_grad("dq", dq, rdq)
    assert sorted(got) == list(range(W))
    for c in range(W):
        _check_grad(f"dk[{c}]", got[c][0], rdkv[c][0])
        _check_grad(f"dv[{c}]", got[c][1], rdkv[c][1])
    _check_grad("own dk", dkv[0], rdkv[rank][0])


def test_bwd_full_size_chunk_properties():
    """The full-size backward shape for one chunk (B1 H32 D128, Q 4096 x 4096 keys): checked on three heads
    against the oracle, and by linearity in dout on all heads: bwd(2 dout) == 2 bwd(dout) up to bf16 rounding."""
    import mercury_artifact_amd as M

    B, Sq, H, D = 1, 4096, 32, 128
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    kv = torch.randn(2, B, Sq, H, D, generator=g).bfloat16()
    dout = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    scale = D ** -0.5
    qd, kvd, dd = q.cuda(), kv.cuda(), dout.cuda()
    od, ld = M.attn_fwd_block(qd, kvd[0], kvd[1], scale)
    dq = torch.empty_like(qd); dkv = torch.empty_like(kvd)
    M.attn_bwd_block(dd, qd, kvd[0], kvd[1], od, ld, dq, dkv[0], dkv[1], scale)
    dq2 = torch.empty_like(qd); dkv2 = torch.empty_like(kvd)
    M.attn_bwd_block(dd * 2, qd, kvd[0], kvd[1], od, ld, dq2, dkv2[0], dkv2[1], scale)
    torch.cuda.synchronize()
    assert _rel(dq2.float(), 2 * dq.float()) <= 1e-2 and _rel(dkv2.float(), 2 * dkv.float()) <= 1e-2
    heads = [0, 13, 31]
    rdq, rdk, rdv = O.block_backward(dout[:, :, heads].float(), q[:, :, heads].float(), kv[0][:, :, heads].float(),
                                     kv[1][:, :, heads].float(), od[:, :, heads].float().cpu(), ld[:, heads].cpu(), scale)
    _check_grad("dq", dq[:, :, heads], rdq)
    _check_grad("dk", dkv[0][:, :, heads], rdk)
    _check_grad("dv", dkv[1][:, :, heads], rdv)


@pytest.mark.parametrize("fused", [True, False])
def test_bwd_ring_full_size(fused):
    """The backward configuration at full size (B1 H32 D128, Q 4096 x 8 KV chunks of 4096): the merged out / LSE
    of the forward ring step feed the backward ring step; dQ accumulated in fp32 over the 8 chunks (inside the
    kernel, or by the literal torch.add sequence) and two chunks' dK / dV are compared on three heads with the
    oracle's ring backward from the same out / LSE."""
    import mercury_artifact_amd as M

    B, Sq, H, D, W, rank = 1, 4096, 32, 128, 8, 5
    g = torch.Generator().manual_seed(9)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    kvs = [torch.randn(2, B, Sq, H, D, generator=g).bfloat16() for _ in range(W)]
    dout = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    scale = D ** -0.5
    dev = [c.cuda() for c in kvs]
    qd, dd = q.cuda(), dout.cuda()
    o = torch.empty_like(qd)
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    M.flash_attn_pack_kv(qd, dev[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev))
    dq = torch.empty_like(qd)
    dkv = torch.empty_like(dev[rank])
    got = {}
    print(f"full-size backward ring, fused_accumulate={fused}", flush=True)
    M.flash_attn_backward(qd, dev[rank], o, lse, dd, dq, dkv, scale, ring=M.LocalRing((W,), rank, dev),
                          dkv_chunks=got, fused_accumulate=fused)
    torch.cuda.synchronize()
    assert sorted(got) == list(range(W))
    heads = [0, 13, 31]
    order = O.single_ring_order(rank, W)
    rdq, rdkv = O.ring_backward(q[:, :, heads].float(), [c[:, :, :, heads].float() for c in kvs], order,
                                o[:, :, heads].float().cpu(), lse[:, heads].cpu(), dout[:, :, heads].float(), scale)
    _check_grad("dq", dq[:, :, heads], rdq)
    for c in (order[0], order[-1]):
        _check_grad(f"dk[{c}]", got[c][0][:, :, heads], rdkv[c][0])
        _check_grad(f"dv[{c}]", got[c][1][:, :, heads], rdkv[c][1])
    assert torch.equal(dkv.float(), got[rank])          # the rank's own chunk is what dkv receives
    # every head: dQ on a window of 256 query rows (a function of those rows alone) over all chunks, and dK / dV of
    # a 256-key window of one chunk (a sum over all query rows)
    rows = slice(2944, 3200)
    wdq, _ = O.ring_backward(q[:, rows].float(), [c.float() for c in kvs], order, o[:, rows].float().cpu(),
                             lse[:, :, rows].cpu(), dout[:, rows].float(), scale)
    _check_grad("dq, all heads", dq[:, rows], wdq)
    c = order[3]
    _, wdkv = O.ring_backward(q.float(), [kvs[c][:, :, 512:768].float()], [0], o.float().cpu(), lse.cpu(),
                              dout.float(), scale)
    _check_grad(f"dk[{c}], all heads", got[c][0][:, 512:768], wdkv[0][0])
    _check_grad(f"dv[{c}], all heads", got[c][1][:, 512:768], wdkv[0][1])


def test_bwd_block_head_dim_64():
    """Head dimension 64 through the backward (the missing columns are zeros on chip only)."""
    import mercury_artifact_amd as M

    q, kv, dout, o16, lse, scale, (rdq, rdk, rdv) = _case(2, 160, 200, 4, 2, True, seed=12, D=64)
    qd, kvd, dd, od, ld = q.cuda(), kv.cuda(), dout.cuda(), o16.cuda(), lse.cuda()
    dq = torch.full_like(qd, float("nan")); dkv = torch.full_like(kvd, float("nan"))
    acc = torch.full(qd.shape, 0.5, dtype=torch.float32, device="cuda")
    M.attn_bwd_block(dd, qd, kvd[0], kvd[1], od, ld, dq, dkv[0], dkv[1], scale, causal=True, dq_acc=acc)
    torch.cuda.synchronize()
    _check_grad("dq", dq, rdq)
    _check_grad("dk", dkv[0], rdk)
    _check_grad("dv", dkv[1], rdv)
    _check_grad("dq_acc", acc - 0.5, rdq)


@pytest.mark.parametrize("D", [64, 24])
def test_bwd_block_small_head_dim_reads_and_writes_only_its_columns(D):
    """Every tensor of the block backward as a column slice of a 128-wide one: NaN next to the inputs, a sentinel
    next to the outputs.  Nothing outside the D columns may be fetched or stored."""
    import mercury_artifact_amd as M

    B, Sq, Sc, Hq, Hkv = 1, 160, 200, 4, 2
    q, kv, dout, o16, lse, scale, (rdq, rdk, rdv) = _case(B, Sq, Sc, Hq, Hkv, False, seed=15, D=D)
    off = 128 - D

    def wide(t, fill):
        w = torch.full(t.shape[:-1] + (128,), fill, dtype=torch.bfloat16, device="cuda")
        w[..., off:].copy_(t.cuda())
        return w, w[..., off:]

    nan = float("nan")
    (_, qv), (_, dv_), (_, ov) = wide(q, nan), wide(dout, nan), wide(o16, nan)
    kvw = torch.full((2, B, Sc, Hkv, 128), nan, dtype=torch.bfloat16, device="cuda")
    kvw[..., off:].copy_(kv.cuda())
    kvv = kvw[..., off:]
    dqw = torch.full((B, Sq, Hq, 128), 7.0, dtype=torch.bfloat16, device="cuda")
    dkvw = torch.full((2, B, Sc, Hkv, 128), 7.0, dtype=torch.bfloat16, device="cuda")
    acc = torch.full((B, Sq, Hq, D), 0.5, dtype=torch.float32, device="cuda")
    M.attn_bwd_block(dv_, qv, kvv[0], kvv[1], ov, lse.cuda(), dqw[..., off:], dkvw[0][..., off:], dkvw[1][..., off:],
                     scale, dq_acc=acc)
    torch.cuda.synchronize()
    _check_grad("dq", dqw[..., off:], rdq)
    _check_grad("dk", dkvw[0][..., off:], rdk)
    _check_grad("dv", dkvw[1][..., off:], rdv)
    _check_grad("dq_acc", acc - 0.5, rdq)
    assert (dqw[..., :off] == 7.0).all() and (dkvw[..., :off] == 7.0).all()


def test_bwd_block_strided_views_without_copies():
    """The call site of the generated backward (utils/attn_bwd_dsl.py:83-115): q / out / dout are views of larger
    buffers (here: a head slice) while block_dq comes from torch.empty, contiguous.  dq and out have stride
    triples of their own in the C ABI, so the operator makes no contiguous copies of anything."""
    import mercury_artifact_amd as M

    B, Sq, Sc, H, D = 1, 192, 256, 2, 128
    g = torch.Generator().manual_seed(14)
    big = {n: torch.randn(B, Sq, 2 * H, D, generator=g).bfloat16() for n in ("q", "dout")}
    kv = torch.randn(2, B, Sc, H, D, generator=g).bfloat16()
    q, dout = big["q"][:, :, H:], big["dout"][:, :, H:]
    scale = D ** -0.5
    o, lse = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale)
    rdq, rdk, rdv = O.block_backward(dout.float(), q.float(), kv[0].float(), kv[1].float(), o.bfloat16().float(), lse, scale)
    qd, dd = big["q"].cuda()[:, :, H:], big["dout"].cuda()[:, :, H:]
    obig = torch.zeros(B, Sq, 3 * H, D, dtype=torch.bfloat16, device="cuda")
    od = obig[:, :, H:2 * H]
    od.copy_(o.bfloat16())
    kvd = kv.cuda()
    dq = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")          # contiguous, like block_dq
    dkv = torch.empty_like(kvd)
    copies = []
    real = torch.Tensor.contiguous

    def spy(self, *a, **kw):
        if not self.is_contiguous():
            copies.append(tuple(self.shape))
        return real(self, *a, **kw)

    torch.Tensor.contiguous = spy
    try:
        M.attn_bwd_block(dd, qd, kvd[0], kvd[1], od, lse.cuda(), dq, dkv[0], dkv[1], scale)
    finally:
        torch.Tensor.contiguous = real
    torch.cuda.synchronize()
    assert copies == []
    _check_grad("dq", dq, rdq)
    _check_grad("dk", dkv[0], rdk)
    _check_grad("dv", dkv[1], rdv)
