"""A ring step replayed as a HIP graph gives, on every replay, exactly what the eager step gives.

Replays are interleaved with eager work and synchronisations, and the inputs change in place between them:
a graph that had frozen stale values, or whose nodes misbehave after the first replay, would fail."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fused,deferred", [(False, False), (True, False), (True, True)])
def test_graphed_single_ring_step_matches_eager(fused, deferred):
    import mercury_artifact_amd as M

    B, S, H, D, W, rank = 2, 256, 4, 128, 4, 1
    scale = D ** -0.5
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn(B, S, H, D, generator=g, device="cuda").bfloat16()
    chunks = [torch.randn(2, B, S, H, D, generator=g, device="cuda").bfloat16() for _ in range(W)]
    o = torch.empty_like(q)
    lse = torch.empty(B, H, S, dtype=torch.float32, device="cuda")

    def step():
        M.flash_attn_pack_kv(q, chunks[rank], o, lse, scale, ring=M.LocalRing((W,), rank, chunks),
                             fused_epilogue=fused, deferred_merge=deferred)

    graphed = M.GraphedStep(step)
    for it in range(4):
        # new inputs, in place
        q.copy_(torch.randn(B, S, H, D, generator=g, device="cuda").bfloat16())
        chunks[(it + 1) % W].copy_(torch.randn(2, B, S, H, D, generator=g, device="cuda").bfloat16())
        step()
        torch.cuda.synchronize()
        eo, el = o.clone(), lse.clone()
        o.zero_()
        lse.zero_()
        (q.float() @ q.float().transpose(-1, -2)).sum().item()      # unrelated eager work + a sync
        graphed.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, eo), it
        assert torch.equal(lse, el), it


def test_graphed_backward_block_matches_eager():
    import mercury_artifact_amd as M

    B, S, H, D = 1, 320, 2, 128
    scale = D ** -0.5
    g = torch.Generator(device="cuda").manual_seed(4)
    q = torch.randn(B, S, H, D, generator=g, device="cuda").bfloat16()
    kv = torch.randn(2, B, S, H, D, generator=g, device="cuda").bfloat16()
    do = torch.randn(B, S, H, D, generator=g, device="cuda").bfloat16()
    o, lse = M.attn_fwd_block(q, kv[0], kv[1], scale, causal=True)
    dq, dkv = torch.empty_like(q), torch.empty_like(kv)

    def step():
        M.attn_bwd_block(do, q, kv[0], kv[1], o, lse, dq, dkv[0], dkv[1], scale, causal=True)

    graphed = M.GraphedStep(step)
    for it in range(3):
        do.copy_(torch.randn(B, S, H, D, generator=g, device="cuda").bfloat16())
        step()
        torch.cuda.synchronize()
        edq, edkv = dq.clone(), dkv.clone()
        dq.zero_()
        dkv.zero_()
        torch.cuda.synchronize()
        graphed.replay()
        torch.cuda.synchronize()
        assert torch.equal(dq, edq) and torch.equal(dkv, edkv), it


def test_search_harness_times_a_step():
    """bench_callable follows the timing protocol of the reference's schedule search: warm-up, timed calls
    between device events, (iterations per second, seconds, bytes)."""
    import mercury_artifact_amd as M
    from mercury_artifact_amd import search_harness as SH

    B, S, H, D, W = 1, 256, 2, 128, 2
    q = torch.randn(B, S, H, D, device="cuda").bfloat16()
    chunks = [torch.randn(2, B, S, H, D, device="cuda").bfloat16() for _ in range(W)]
    o = torch.zeros_like(q)
    lse = torch.zeros(B, H, S, dtype=torch.float32, device="cuda")

    def step(q, kv, o, lse):
        M.flash_attn_pack_kv(q, kv, o, lse, D ** -0.5, ring=M.LocalRing((W,), 0, chunks))

    ips, seconds, nbytes = SH.bench_callable(step, {"q": q, "kv": chunks[0], "o": o, "lse": lse}, num_iter=5)
    assert ips > 0 and seconds > 0 and abs(ips * seconds - 5) < 1e-6
    assert nbytes == sum(t.numel() * t.element_size() for t in (q, chunks[0], o, lse))
    assert o.float().abs().max().item() > 0
    with pytest.raises(ImportError):
        SH.bench_program(object())          # the IR and its code generator are not part of this package


@pytest.mark.parametrize("lazy", [False, True])
def test_search_harness_bench_program_allocates_execs_and_times(lazy, capsys):
    """bench_program end to end without the reference's package: a stand-in program (name + I/O buffers) and a
    Lowering whose generator returns this repo's generated-style step text.  The harness must exec the text in a
    namespace holding this package's operators, allocate zeros for written buffers and N(0,1) for the others in
    the buffers' dtypes, run warm-up and timed calls, and report the program's buffer bytes."""
    import types

    import mercury_artifact_amd as M
    from mercury_artifact_amd import search_harness as SH
    from test_gpu_generated_style import SINGLE_RING_TEXT, _Dist

    B, S, H, D, W, rank = 1, 256, 2, 128, 2, 1
    Buf = types.SimpleNamespace
    buffers = [Buf(tensor="q", shape=(B, S, H, D), dtype=torch.bfloat16, write=False),
               Buf(tensor="kv", shape=(2, B, S, H, D), dtype=torch.bfloat16, write=False),
               Buf(tensor="o", shape=(B, S, H, D), dtype=torch.bfloat16, write=True),
               Buf(tensor="lse", shape=(B, H, S), dtype=torch.float32, write=True)]
    program = Buf(name="ring_step", buffers=buffers, eliminated=False)
    nbytes = sum(torch.empty(b.shape, dtype=b.dtype).numel() * torch.empty((), dtype=b.dtype).element_size() for b in buffers)
    seen = {}

    def generate(prog):
        assert prog.eliminated                       # loops are eliminated before the text is generated
        return SINGLE_RING_TEXT

    low = SH.Lowering(eliminate_loops=lambda prog: setattr(prog, "eliminated", True), generate_code=generate,
                      io_buffers=lambda prog: prog.buffers, buffer_bytes=lambda prog: nbytes)
    other = [torch.randn(2, B, S, H, D, device="cuda").bfloat16() for _ in range(W)]

    class Ring(M.LocalRing):                         # the hop of the generated loop, and a look at the arguments
        def __init__(self):
            super().__init__((W,), rank, other)

        def send_recv(self, send_to, recv_from, tensor):
            seen.setdefault("kv_dtype", tensor.dtype)
            return super().send_recv(send_to, recv_from, tensor)

    extra = {"torch": torch, "dist": _Dist(rank), "WORLD": W, "SendRecv": Ring}
    real_bench_callable = SH.bench_callable

    def spy(func, call, *a, **kw):                   # the tensors the harness allocated
        seen["call"] = call
        return real_bench_callable(func, call, *a, **kw)

    SH.bench_callable = spy
    try:
        ips, seconds, mem = SH.bench_program(program, extra, num_iter=3, kwargs={"softmax_scale": D ** -0.5},
                                             log=True, lowering=low, lazy_merge=lazy)
    finally:
        SH.bench_callable = real_bench_callable
    assert ips > 0 and seconds > 0 and abs(ips * seconds - 3) < 1e-6 and mem == nbytes
    assert seen["kv_dtype"] == torch.bfloat16
    # what the timed function left in the output buffers is the ring step of the oracle on the allocated inputs
    call = seen["call"]
    assert call["q"].dtype == torch.bfloat16 and call["lse"].dtype == torch.float32
    chunks = [c.float().cpu() for c in other]
    chunks[rank] = call["kv"].float().cpu()
    import oracle as O
    ro, rl = O.ring_forward(call["q"].float().cpu(), chunks, O.single_ring_order(rank, W), D ** -0.5)
    assert (call["o"].float().cpu() - ro).abs().max().item() <= 2e-2
    assert ((call["lse"].cpu() - rl).abs() / rl.abs().clamp_min(1.0)).max().item() <= 1e-3
    printed = capsys.readouterr().out
    assert "def ring_step" in printed and "iter/s" in printed and "Memory cost" in printed


def test_graphed_fp8_step_matches_eager():
    """The fp8 step takes its three descales as device scalars that the kernel reads when it runs: the step is
    captured without any device-to-host copy, replays bit-identically, and a replay after the scales were rewritten
    in place (the normal case of re-quantising every step) uses the new values, as the eager step does."""
    import mercury_artifact_amd as M

    B, S, H, D, W, rank = 1, 256, 2, 128, 2, 1
    scale = D ** -0.5
    g = torch.Generator(device="cuda").manual_seed(6)
    (q8, sq) = M.quantize_e4m3(torch.randn(B, S, H, D, generator=g, device="cuda"))
    k8, sk = M.quantize_e4m3(torch.randn(W, B, S, H, D, generator=g, device="cuda"))
    v8, sv = M.quantize_e4m3(torch.randn(W, B, S, H, D, generator=g, device="cuda"))
    chunks = [torch.stack([k8[c], v8[c]]) for c in range(W)]
    o = torch.empty(B, S, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, S, dtype=torch.float32, device="cuda")

    def step():
        M.fp8_pack_split_kv(q8, chunks[rank], o, lse, scale, sq, sk, sv, ring=M.LocalRing((W,), rank, chunks))

    graphed = M.GraphedStep(step)
    for it in range(3):
        step()
        torch.cuda.synchronize()
        eo, el = o.clone(), lse.clone()
        o.zero_()
        lse.zero_()
        torch.cuda.synchronize()
        graphed.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, eo) and torch.equal(lse, el), it
    # descales rewritten in place between replays: by a torch op, and through the raw pointer (a write no version
    # counter sees); eager call and replay both read the value that is in memory when the kernel runs
    before_o, before_l = o.clone(), lse.clone()
    sv.mul_(2.0)
    step()
    torch.cuda.synchronize()
    assert torch.allclose(o.float(), 2.0 * before_o.float(), rtol=2 ** -7, atol=1e-6) and torch.equal(lse, before_l)
    o.zero_()
    graphed.replay()
    torch.cuda.synchronize()
    assert torch.allclose(o.float(), 2.0 * before_o.float(), rtol=2 ** -7, atol=1e-6)
    sq.mul_(0.5)
    step()
    torch.cuda.synchronize()
    eo, el = o.clone(), lse.clone()
    assert not torch.equal(el, before_l)
    o.zero_()
    lse.zero_()
    graphed.replay()
    torch.cuda.synchronize()
    assert torch.equal(o, eo) and torch.equal(lse, el)
    import ctypes
    half = (ctypes.c_float * 1)(float(sk) * 0.5)
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    assert hip.hipMemcpy(sk.data_ptr(), ctypes.addressof(half), 4, 1) == 0        # 1 = host to device
    torch.cuda.synchronize()
    step()
    torch.cuda.synchronize()
    eo2, el2 = o.clone(), lse.clone()
    assert not torch.equal(el2, el)
    o.zero_()
    lse.zero_()
    graphed.replay()
    torch.cuda.synchronize()
    assert torch.equal(o, eo2) and torch.equal(lse, el2)
