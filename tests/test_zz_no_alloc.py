"""mhip_attn_bwd_block_noalloc: the block backward with its workspace in a device array built into the library
(for callers that cannot allocate).  It shares its kernels with mhip_attn_bwd_block, so the results must be
bit-identical to that entry point's: integer comparison of the bf16 / fp32 bit patterns, on two calls in a
row, the second one smaller (the scratch keeps the first call's contents)."""
import pytest
import torch

from mercury_artifact_amd import _native as N

pytestmark = pytest.mark.gpu
ETOOLARGE = -7


def _inputs(B, Sq, Sc, Hq, Hkv, seed, D=128):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *shape: torch.randn(*shape, generator=g).bfloat16().cuda()
    q, dout = mk(B, Sq, Hq, D), mk(B, Sq, Hq, D)
    kv = mk(2, B, Sc, Hkv, D)
    return q, kv[0], kv[1], dout


def _call(entry, q, k, v, out, lse, dout, scale, causal, with_acc):
    B, Sq, Hq, D = q.shape
    Sc, Hkv = k.shape[1], k.shape[2]
    dq = torch.full_like(q, float("nan"))
    dkv = torch.full((2,) + tuple(k.shape), float("nan"), dtype=k.dtype, device=k.device)
    dq_acc = torch.full(q.shape, 0.25, dtype=torch.float32, device=q.device) if with_acc else None
    args = [N.ptr(dout), N.ptr(q), N.ptr(k), N.ptr(v), N.ptr(out), N.ptr(lse), N.ptr(dq), N.ptr(dkv[0]), N.ptr(dkv[1]),
            N.ptr(dq_acc), B, Sq, Sc, Hq, Hkv, D, q.stride(0), q.stride(1), q.stride(2),
            k.stride(0), k.stride(1), k.stride(2), dkv[0].stride(0), dkv[0].stride(1), dkv[0].stride(2),
            dq.stride(0), dq.stride(1), dq.stride(2), out.stride(0), out.stride(1), out.stride(2),
            scale, 1 if causal else 0, 0]
    stream = N.stream_of(q)
    if entry == "workspace":
        ws = torch.empty(N.lib().mhip_attn_bwd_workspace_bytes(B, Sq, Sc, Hq, Hkv, D), dtype=torch.uint8, device=q.device)
        code = N.lib().mhip_attn_bwd_block(*args, N.ptr(ws), stream)
    else:
        code = N.lib().mhip_attn_bwd_block_noalloc(*args, stream)
    N.check(code, entry)
    torch.cuda.synchronize()
    return dq, dkv, dq_acc


def _bits(t):
    return t.view(torch.int16) if t.dtype == torch.bfloat16 else t.view(torch.int32)


@pytest.mark.parametrize("causal", [False, True])
def test_no_alloc_entry_matches_the_workspace_entry(causal):
    import mercury_artifact_amd as M

    scale = 128 ** -0.5
    # two calls in a row, the second with a smaller input; GQA in the first
    for (B, Sq, Sc, Hq, Hkv, seed, with_acc) in ((2, 384, 320, 4, 2, 1, True), (1, 100, 77, 2, 2, 2, False)):
        print(f"no-alloc case B{B} Sq{Sq} Sc{Sc} Hq{Hq} Hkv{Hkv} causal={causal}", flush=True)
        q, k, v, dout = _inputs(B, Sq, Sc, Hq, Hkv, seed)
        out, lse = M.attn_fwd_block(q, k, v, scale, causal=causal)
        got = _call("noalloc", q, k, v, out, lse, dout, scale, causal, with_acc)
        want = _call("workspace", q, k, v, out, lse, dout, scale, causal, with_acc)
        for name, a, b in zip(("dq", "dkv", "dq_acc"), got, want):
            if a is None:
                assert b is None
                continue
            assert not torch.isnan(a.float()).any(), name
            assert torch.equal(_bits(a), _bits(b)), name


def test_no_alloc_entry_rejects_what_does_not_fit():
    q, k, v, dout = _inputs(1, 64, 64, 2, 2, 3)
    lib = N.lib()
    P = N.ptr(q)
    # 2^20 + 1 rows: refused before anything is launched (the pointers are never used)
    code = lib.mhip_attn_bwd_block_noalloc(P, P, P, P, P, P, P, P, P, None, 1, (1 << 20) + 1, 64, 1, 1, 128,
                                           ((1 << 20) + 1) * 128, 128, 128, 64 * 128, 128, 128, 64 * 128, 128, 128,
                                           ((1 << 20) + 1) * 128, 128, 128, ((1 << 20) + 1) * 128, 128, 128,
                                           0.1, 0, 0, None)
    assert code == ETOOLARGE
    assert b"scratch" in lib.mhip_error_string(code)


def test_no_alloc_entry_recorded_into_a_hip_graph():
    """The use it is meant for: after mhip_init() (the symbol-address query, outside the capture) the call is
    recorded into a HIP graph; every replay, with the program's own eager work and synchronisations in between
    and the inputs rewritten in place, gives the bits of an eager call on the same inputs."""
    import mercury_artifact_amd as M

    scale = 128 ** -0.5
    B, Sq, Sc, Hq, Hkv = 1, 256, 192, 4, 2
    q, k, v, dout = _inputs(B, Sq, Sc, Hq, Hkv, 5)
    out, lse = M.attn_fwd_block(q, k, v, scale)
    dq = torch.empty_like(q)
    dkv = torch.empty((2,) + tuple(k.shape), dtype=k.dtype, device=k.device)
    assert N.lib().mhip_init() == 0

    def call():
        args = [N.ptr(dout), N.ptr(q), N.ptr(k), N.ptr(v), N.ptr(out), N.ptr(lse), N.ptr(dq), N.ptr(dkv[0]), N.ptr(dkv[1]),
                None, B, Sq, Sc, Hq, Hkv, 128, q.stride(0), q.stride(1), q.stride(2),
                k.stride(0), k.stride(1), k.stride(2), dkv[0].stride(0), dkv[0].stride(1), dkv[0].stride(2),
                dq.stride(0), dq.stride(1), dq.stride(2), out.stride(0), out.stride(1), out.stride(2), scale, 0, 0]
        N.check(N.lib().mhip_attn_bwd_block_noalloc(*args, N.stream_of(q)), "noalloc")

    graphed = M.GraphedStep(call, warmup=0)          # recorded without an eager call before it
    for it in range(3):
        if it:                                        # new inputs, in place
            g = torch.Generator().manual_seed(50 + it)
            dout.copy_(torch.randn(dout.shape, generator=g).bfloat16())
        torch.cuda.synchronize()
        call()
        torch.cuda.synchronize()
        want = (dq.clone(), dkv.clone())
        dq.zero_()
        dkv.zero_()
        torch.cuda.synchronize()
        graphed.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(dq), _bits(want[0])) and torch.equal(_bits(dkv), _bits(want[1])), it
