"""Seeded random small shapes through the three block kernels and the one-pass fold against the CPU oracle: ragged row and key
counts, batch 1-3, 1-4 query heads per KV head, with and without the causal mask, and (bf16) a head dimension drawn
from the multiples of 8 up to 128, half of the cases 128.  Tolerances as in the per-kernel test files."""
import random

import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu


def _shapes(seed, n, max_s):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        hkv = rng.randint(1, 2)
        out.append((rng.randint(1, 3), rng.randint(1, max_s), rng.randint(1, max_s), hkv * rng.randint(1, 4), hkv,
                    rng.random() < 0.5))
    return out


def _head_dim(*key):
    seed = 0
    for k in key:
        seed = seed * 1000003 + int(k)
    rng = random.Random(seed)
    return 128 if rng.random() < 0.5 else 8 * rng.randint(1, 15)


@pytest.mark.parametrize("B,Sq,Sc,Hq,Hkv,causal", _shapes(101, 16, 420))
def test_random_forward(B, Sq, Sc, Hq, Hkv, causal):
    import mercury_artifact_amd as M

    D = _head_dim(B, Sq, Sc, Hq)
    print(f"fwd B{B} Sq{Sq} Sc{Sc} Hq{Hq} Hkv{Hkv} D{D} causal={causal}", flush=True)
    g = torch.Generator().manual_seed(B * 1000003 + Sq * 1009 + Sc)
    q = torch.randn(B, Sq, Hq, D, generator=g).bfloat16()
    kv = torch.randn(2, B, Sc, Hkv, D, generator=g).bfloat16()
    scale = D ** -0.5
    ro, rl = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale, causal=causal)
    out, lse = M.attn_fwd_block(q.cuda(), kv[0].cuda(), kv[1].cuda(), scale, causal=causal)
    out, lse = out.float().cpu(), lse.cpu()
    assert torch.equal(torch.isinf(lse), torch.isinf(rl))
    assert (out - ro).abs().max().item() <= 2e-2
    if ro.norm().item() > 0:
        assert (out - ro).norm().item() / ro.norm().item() <= 1e-2
    fin = ~torch.isinf(rl)
    if fin.any():
        assert ((lse[fin] - rl[fin]).abs() / rl[fin].abs().clamp_min(1.0)).max().item() <= 1e-3


@pytest.mark.parametrize("B,Sq,Sc,Hq,Hkv,causal", _shapes(202, 12, 300))
def test_random_backward(B, Sq, Sc, Hq, Hkv, causal):
    import mercury_artifact_amd as M

    D = _head_dim(B, Sq, Sc, Hq, 7)
    print(f"bwd B{B} Sq{Sq} Sc{Sc} Hq{Hq} Hkv{Hkv} D{D} causal={causal}", flush=True)
    g = torch.Generator().manual_seed(B * 1000003 + Sq * 1009 + Sc + 7)
    q = torch.randn(B, Sq, Hq, D, generator=g).bfloat16()
    kv = torch.randn(2, B, Sc, Hkv, D, generator=g).bfloat16()
    dout = torch.randn(B, Sq, Hq, D, generator=g).bfloat16()
    scale = D ** -0.5
    o, lse = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale, causal=causal)
    o16 = o.bfloat16()
    refs = O.block_backward(dout.float(), q.float(), kv[0].float(), kv[1].float(), o16.float(), lse, scale,
                            causal=causal)
    qd, kvd = q.cuda(), kv.cuda()
    dq = torch.full_like(qd, float("nan"))
    dkv = torch.full_like(kvd, float("nan"))
    M.attn_bwd_block(dout.cuda(), qd, kvd[0], kvd[1], o16.cuda(), lse.cuda(), dq, dkv[0], dkv[1], scale, causal=causal)
    for name, got, ref in (("dq", dq, refs[0]), ("dk", dkv[0], refs[1]), ("dv", dkv[1], refs[2])):
        got = got.float().cpu()
        assert not torch.isnan(got).any(), name
        scale_ref = ref.abs().max().item()
        assert (got - ref).abs().max().item() <= 4e-2 * scale_ref + 1e-6, name
        if ref.norm().item() > 1e-3:
            assert (got - ref).norm().item() / ref.norm().item() <= 1.5e-2, name


@pytest.mark.parametrize("B,Sq,Sc,Hq,Hkv,causal", _shapes(303, 10, 500))
def test_random_fp8_forward(B, Sq, Sc, Hq, Hkv, causal):
    import mercury_artifact_amd as M

    print(f"fp8 B{B} Sq{Sq} Sc{Sc} Hq{Hq} Hkv{Hkv} causal={causal}", flush=True)
    g = torch.Generator().manual_seed(B * 1000003 + Sq * 1009 + Sc + 13)
    q = torch.randn(B, Sq, Hq, 128, generator=g)
    k = torch.randn(B, Sc, Hkv, 128, generator=g)
    v = torch.randn(B, Sc, Hkv, 128, generator=g)
    (qq, sq), (kq, sk), (vq, sv) = O.quantize_e4m3(q), O.quantize_e4m3(k), O.quantize_e4m3(v)
    scale = 128 ** -0.5
    oa, la = O.block_attention(O.dequantize(qq, sq), O.dequantize(kq, sk), O.dequantize(vq, sv), scale, causal=causal)
    out, lse = M.attn_fwd_block(qq.cuda(), kq.cuda(), vq.cuda(), scale, causal=causal,
                                q_descale=sq.cuda(), k_descale=sk.cuda(), v_descale=sv.cuda())
    out, lse = out.float().cpu(), lse.cpu()
    assert torch.equal(torch.isinf(lse), torch.isinf(la))
    # per element within what rounding P to e4m3 can do (2^-4 times attention over |v|: few visible keys and
    # large |v| make that larger than any fixed number) plus one bf16 rounding of the result and 2e-3
    p_bound = O.e4m3_p_rounding_bound(O.dequantize(qq, sq), O.dequantize(kq, sk), O.dequantize(vq, sv), scale,
                                      causal=causal)
    assert ((out - oa).abs() - (p_bound + 2 ** -8 * oa.abs() + 2e-3)).max().item() <= 0
    if oa.norm().item() > 0:
        assert (out - oa).norm().item() / oa.norm().item() <= 6e-2
    fin = ~torch.isinf(la)
    if fin.any():
        assert ((lse[fin] - la[fin]).abs() / la[fin].abs().clamp_min(1.0)).max().item() <= 1e-3


def _fold_cases(seed, n):
    rng = random.Random(seed)
    return [(rng.randint(1, 3), rng.randint(1, 300), rng.randint(1, 6), rng.choice([64, 128, 256, 128, 96, 40, 8, 200]), rng.randint(1, 16))
            for _ in range(n)]


@pytest.mark.parametrize("B,Sq,H,D,n", _fold_cases(404, 12))
def test_random_fold_of_block_results(B, Sq, H, D, n):
    """merge_many on random shapes and block counts, some blocks covering only a tail of the rows, against the
    chain of reference merges in fp64 (bf16 result: atol 1e-3 + rtol 2^-8; lse 1e-5)."""
    import mercury_artifact_amd as M

    print(f"fold B{B} Sq{Sq} H{H} D{D} n{n}", flush=True)
    rng = random.Random(B * 7919 + Sq * 31 + n)
    g = torch.Generator().manual_seed(B * 1000003 + Sq * 1009 + n)
    begins = [0] + [rng.choice([0, 0, rng.randint(0, Sq)]) for _ in range(n - 1)]
    outs = [torch.randn(B, Sq - sb, H, D, generator=g).bfloat16() for sb in begins]
    lses = [torch.randn(B, H, Sq - sb, generator=g) * 4 for sb in begins]
    out = lse = None
    for bo, bl, sb in zip(outs, lses, begins):
        if bo.shape[1] == 0:
            continue
        sl = None if sb == 0 else (slice(None), slice(sb, None))
        out, lse = O.update_out_and_lse(out, lse, bo, bl, slice_=sl, acc_dtype=torch.float64)
    ro, rl = out.float(), lse.squeeze(-1).transpose(1, 2).float()
    fo = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    fl = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    M.merge_many([t.cuda() for t in outs], [t.cuda() for t in lses], fo, fl, row_begin=begins)
    assert ((fo.float().cpu() - ro).abs() - (1e-3 + 2 ** -8 * ro.abs())).max().item() <= 0
    assert ((fl.cpu() - rl).abs() / rl.abs().clamp_min(1.0)).max().item() <= 1e-5
