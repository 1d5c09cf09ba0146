"""Ring-step drivers on one GPU against the CPU oracle's ring step on the same seeded inputs.

Same tolerances as the block kernel (bf16: max-abs(out) <= 2e-2, LSE rel <= 1e-3, own rel-L2 <= 1e-2);
the reference's own tests accept max-abs < 1e-2 on out and lse (tests/test_search_validation.py:207-208),
which is asserted too at the reference's test shape."""
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu


def _inputs(B, S, Hq, Hkv, D, W, seed=0):
    """Full-sequence q, k, v (N(0,1) -> bf16) and the per-rank shards the reference's tests make with
    ``chunk(W, dim=1)`` (example.py:161)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, S, Hq, D, generator=g).bfloat16()
    k = torch.randn(B, S, Hkv, D, generator=g).bfloat16()
    v = torch.randn(B, S, Hkv, D, generator=g).bfloat16()
    Sc = S // W
    qs = [q[:, r * Sc:(r + 1) * Sc] for r in range(W)]
    kvs = [torch.stack([k[:, r * Sc:(r + 1) * Sc], v[:, r * Sc:(r + 1) * Sc]]) for r in range(W)]
    return q, k, v, qs, kvs


def _compare(o, lse, ro, rl, out_atol=2e-2, lse_rtol=1e-3, rel_l2=1e-2):
    o, lse = o.float().cpu(), lse.float().cpu()
    assert (o - ro).abs().max().item() <= out_atol
    assert (o - ro).norm().item() / ro.norm().item() <= rel_l2
    assert ((lse - rl).abs() / rl.abs().clamp_min(1.0)).max().item() <= lse_rtol


@pytest.mark.parametrize("rank", [0, 5])
@pytest.mark.parametrize("fused,deferred", [(False, False), (True, False), (True, True)])
def test_single_ring_reference_test_shape(rank, fused, deferred):
    """B4 S4096 H5 D128 on an 8-rank ring (tests/test_ring_attn_codegen.py:84-87), one rank."""
    import mercury_artifact_amd as M

    B, S, H, D, W = 4, 4096, 5, 128, 8
    q, k, v, qs, kvs = _inputs(B, S, H, H, D, W)
    scale = D ** -0.5
    ro, rl = O.single_pass_attention(qs[rank].float(), k.float(), v.float(), scale)
    ring_o, ring_l = O.ring_forward(qs[rank].float(), [c.float() for c in kvs],
                                    O.single_ring_order(rank, W), scale)
    assert torch.allclose(ring_o, ro, atol=1e-5)           # oracle ring == oracle single pass
    dev_kvs = [c.cuda() for c in kvs]
    ring = M.LocalRing((W,), rank, dev_kvs)
    qd = qs[rank].cuda()
    o = torch.empty_like(qd)
    lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
    q_before, kv_before = qd.clone(), dev_kvs[rank].clone()
    M.flash_attn_pack_kv(qd, dev_kvs[rank], o, lse, scale, ring=ring, fused_epilogue=fused, deferred_merge=deferred)
    torch.cuda.synchronize()
    _compare(o, lse, ring_o, ring_l)
    assert (o.float().cpu() - ro).abs().max().item() < 1e-2 and (lse.cpu() - rl).abs().max().item() < 1e-2
    assert torch.equal(qd, q_before) and torch.equal(dev_kvs[rank], kv_before)   # inputs untouched


@pytest.mark.parametrize("D", [96, 40, 64])
@pytest.mark.parametrize("deferred", [True, False])
def test_single_ring_other_head_dims(D, deferred):
    """The ring drivers at head dimensions other than 128: block kernels on zero-filled on-chip columns, the fold
    (or the chain of merges) on D-wide rows."""
    import mercury_artifact_amd as M

    B, S, H, W, rank = 2, 1024, 3, 4, 2
    q, k, v, qs, kvs = _inputs(B, S, H, H, D, W, seed=9)
    scale = D ** -0.5
    ro, rl = O.single_pass_attention(qs[rank].float(), k.float(), v.float(), scale)
    dev_kvs = [c.cuda() for c in kvs]
    qd = qs[rank].cuda()
    o = torch.empty_like(qd)
    lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
    M.flash_attn_pack_kv(qd, dev_kvs[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev_kvs),
                         deferred_merge=deferred, fused_epilogue=deferred)
    torch.cuda.synchronize()
    _compare(o, lse, ro, rl)


@pytest.mark.parametrize("divide,deferred", [(2, True), (4, True), (4, False), (8, True), (16, True)])
def test_single_ring_with_ring_divide(divide, deferred):
    """ring_divide = k (tests/test_ring_attn_codegen.py:102, benchmark/bench_attn.py:178): k * W block calls on
    sub-chunks in the order of the generated loops; the result is attention over all keys."""
    import mercury_artifact_amd as M

    B, S, H, D, W, rank = 2, 2048, 3, 128, 4, 3
    q, k, v, qs, kvs = _inputs(B, S, H, H, D, W, seed=5)
    scale = D ** -0.5
    sub = S // W // divide
    subchunks = {(c, s): kvs[c][:, :, s * sub:(s + 1) * sub].float() for c in range(W) for s in range(divide)}
    order = O.ring_divide_order(rank, W, divide)
    keys = list(subchunks)
    ro, rl = O.ring_forward(qs[rank].float(), [subchunks[key] for key in keys], [keys.index(x) for x in order], scale)
    so, sl = O.single_pass_attention(qs[rank].float(), k.float(), v.float(), scale)
    assert torch.allclose(ro, so, atol=1e-5)
    dev = [c.cuda() for c in kvs]
    o = torch.empty(B, S // W, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
    from mercury_artifact_amd import flash_attn_interface as FI

    calls = []
    real = FI.attn_fwd_block

    def counted(q_, k_, *a, **kw):
        calls.append(tuple(k_.shape))
        return real(q_, k_, *a, **kw)

    FI.attn_fwd_block = counted
    try:
        M.flash_attn_pack_kv(qs[rank].cuda(), dev[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev),
                             ring_divide=divide, deferred_merge=deferred)
    finally:
        FI.attn_fwd_block = real
    assert calls == [(B, sub, H, D)] * (W * divide)
    _compare(o, lse, ro, rl)
    with pytest.raises(ValueError):
        M.flash_attn_pack_kv(qs[rank].cuda(), dev[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev),
                             ring_divide=7)


def test_ring_divide_beyond_the_fold_limit_warns_and_merges_block_by_block():
    """128 blocks (ring_divide 32 on 4 ranks) exceed what one fold takes: the driver says so and merges block by
    block; the result is the same attention over all keys."""
    import mercury_artifact_amd as M

    B, S, H, D, W, rank, divide = 1, 2048, 2, 128, 4, 1, 32
    q, k, v, qs, kvs = _inputs(B, S, H, H, D, W, seed=6)
    scale = D ** -0.5
    so, sl = O.single_pass_attention(qs[rank].float(), k.float(), v.float(), scale)
    dev = [c.cuda() for c in kvs]
    o = torch.empty(B, S // W, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
    assert W * divide > M.merge.MAX_MERGE_MANY
    with pytest.warns(RuntimeWarning, match="merges block by block"):
        M.flash_attn_pack_kv(qs[rank].cuda(), dev[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev),
                             ring_divide=divide)
    _compare(o, lse, so, sl)


def test_gqa_ring():
    """Hq 32 / Hkv 8 (tests/test_gqa.py:25), shortened sequence."""
    import mercury_artifact_amd as M

    B, S, Hq, Hkv, D, W, rank = 1, 2048, 32, 8, 128, 4, 2
    q, k, v, qs, kvs = _inputs(B, S, Hq, Hkv, D, W, seed=1)
    scale = D ** -0.5
    ro, rl = O.ring_forward(qs[rank].float(), [c.float() for c in kvs], O.single_ring_order(rank, W), scale)
    dev = [c.cuda() for c in kvs]
    o = torch.empty(B, S // W, Hq, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, Hq, S // W, dtype=torch.float32, device="cuda")
    M.gqa_pack_kv(qs[rank].cuda(), dev[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev))
    _compare(o, lse, ro, rl)


@pytest.mark.parametrize("rank", [0, 6])
def test_double_ring(rank):
    """(inner, outer) = (4, 2) mesh (tests/test_double_ring.py:56)."""
    import mercury_artifact_amd as M

    B, S, H, D, W = 1, 2048, 4, 128, 8
    q, k, v, qs, kvs = _inputs(B, S, H, H, D, W, seed=2)
    scale = D ** -0.5
    order = O.double_ring_order(rank, 4, 2)
    ro, rl = O.ring_forward(qs[rank].float(), [c.float() for c in kvs], order, scale)
    dev = [c.cuda() for c in kvs]
    ring = M.LocalRing((4, 2), rank, dev)
    seen = []
    real_send = ring.send_recv

    def spy(*a, **kw):
        got = real_send(*a, **kw)
        seen.append(ring.current)
        return got
    ring.send_recv = spy
    o = torch.empty(B, S // W, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
    M.flash_attn_pack_split_kv(qs[rank].cuda(), dev[rank], o, lse, scale, ring=ring)
    assert [rank] + seen == order
    _compare(o, lse, ro, rl)


@pytest.mark.parametrize("fused", [False, True])
def test_packed_reduce_ring(fused):
    import mercury_artifact_amd as M

    B, S, H, D, W, rank = 2, 1024, 3, 128, 4, 1
    q, k, v, qs, kvs = _inputs(B, S, H, H, D, W, seed=3)
    scale = D ** -0.5
    ro, rl = O.ring_forward_packed(qs[rank].float(), [c.float() for c in kvs], O.single_ring_order(rank, W), scale)
    dev = [c.cuda() for c in kvs]
    o = torch.empty(B, S // W, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
    M.flash_attn_expose_reduce(qs[rank].cuda(), dev[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev),
                               fused_epilogue=fused)
    _compare(o, lse, ro, rl)


@pytest.mark.parametrize("deferred", [False, True])
@pytest.mark.parametrize("rank", [0, 1, 3])
def test_zigzag_causal_ring(rank, deferred):
    """Causal GQA in the zigzag layout, a scaled-down Llama-3-8B shape (B2, Hq/Hkv = 4, D128)."""
    import mercury_artifact_amd as M

    B, Hq, Hkv, D, W, block = 2, 8, 2, 128, 4, 192
    S = 2 * W * block
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, S, Hq, D, generator=g).bfloat16()
    k = torch.randn(B, S, Hkv, D, generator=g).bfloat16()
    v = torch.randn(B, S, Hkv, D, generator=g).bfloat16()
    scale = D ** -0.5
    ref_o, ref_l = O.single_pass_attention(q.float(), k.float(), v.float(), scale, causal=True)
    pos = [O.zigzag_local_positions(r, W, block) for r in range(W)]
    dev = [torch.stack([k[:, p], v[:, p]]).cuda() for p in pos]
    qd = q[:, pos[rank]].cuda()
    o = torch.empty_like(qd)
    lse = torch.empty(B, Hq, 2 * block, dtype=torch.float32, device="cuda")
    M.zigzag_causal_pack_kv(qd, dev[rank], o, lse, scale, ring=M.LocalRing((W,), rank, dev),
                            deferred_merge=deferred)
    _compare(o, lse, ref_o[:, pos[rank]], ref_l[:, :, pos[rank]])


@pytest.mark.parametrize("mesh", [(4,), (4, 2)])
def test_reduce_buffer_ring_all_ranks(mesh):
    """Managed reduction scheduled as a ring over the packed partial result: Q and (out | lse) travel, KV
    stays; after the write-back hop every rank must hold attention of its own Q rows over ALL keys."""
    import mercury_artifact_amd as M

    W = 1
    for m in mesh:
        W *= m
    B, S, H, D = 1, 128 * W, 2, 128
    q, k, v, qs, kvs = _inputs(B, S, H, H, D, W, seed=6)
    scale = D ** -0.5
    ref_o, ref_l = O.single_pass_attention(q.float(), k.float(), v.float(), scale)
    Sc = S // W
    qd = [x.cuda() for x in qs]
    kvd = [x.cuda() for x in kvs]
    outs = [torch.empty(B, Sc, H, D, dtype=torch.bfloat16, device="cuda") for _ in range(W)]
    lses = [torch.empty(B, H, Sc, dtype=torch.float32, device="cuda") for _ in range(W)]
    M.flash_attn_expose_reduce_q_ring(qd, kvd, outs, lses, scale, mesh_shape=mesh)
    torch.cuda.synchronize()
    for r in range(W):
        _compare(outs[r], lses[r], ref_o[:, r * Sc:(r + 1) * Sc], ref_l[:, :, r * Sc:(r + 1) * Sc])


@pytest.mark.parametrize("copy", [False, True])
@pytest.mark.parametrize("ring_divide", [1, 2])
def test_two_stream_step_is_bit_identical(copy, ring_divide):
    """``two_streams=True`` sends every other block launch to a second stream.  Same kernels on the same operands,
    one fold: the step has to give the single-stream result bit for bit, also when the hops copy the chunks (a block on
    the second stream then has to wait for the copy that delivers its chunk) and with sub-chunk loops; repeated, so
    that a launch that ran ahead of its operand would show."""
    import mercury_artifact_amd as M

    B, S, H, D, W, rank = 1, 512, 4, 128, 4, 1
    g = torch.Generator(device="cuda").manual_seed(17)
    q = torch.randn(B, S, H, D, generator=g, device="cuda").bfloat16()
    kvs = [torch.randn(2, B, S, H, D, generator=g, device="cuda").bfloat16() for _ in range(W)]
    scale = D ** -0.5

    def step(two):
        o = torch.empty_like(q)
        lse = torch.empty(B, H, S, dtype=torch.float32, device="cuda")
        M.flash_attn_pack_kv(q, kvs[rank], o, lse, scale, ring=M.LocalRing((W,), rank, kvs, copy=copy),
                             ring_divide=ring_divide, two_streams=two)
        return o, lse

    ref_o, ref_l = step(False)
    for _ in range(5):
        o, lse = step(True)
        torch.cuda.synchronize()
        assert torch.equal(o, ref_o) and torch.equal(lse, ref_l)
    ro, rl = O.ring_forward(q.float().cpu(), [c.float().cpu() for c in kvs], O.single_ring_order(rank, W), scale)
    assert (ref_o.float().cpu() - ro).abs().max().item() <= 2e-2
