"""Drop-in check of the name-resolution boundary: a function written the way Mercury's generator spells a
ring step (bare names looked up in the dict the text is exec-ed in, keyword-only block call built from
``get_default_args(...).copy()``, ``SendRecv`` protocol, epilogue copies) runs unchanged against
``mercury_artifact_amd.namespace()`` and matches the CPU oracle.  The text below is this repo's own; the
structure follows mercury/backend/pytorch/codegen.py:196-199, 250-252, 264-355, 442-523."""
import os

import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

SINGLE_RING_TEXT = '''
def ring_step(q, kv, o, lse, softmax_scale, dropout_p=0, causal=False, window_size=(-1, -1),
              alibi_slopes=None, deterministic=False):
    indices = one_dim_to_n_dim(dist.get_rank(), (WORLD,))
    assert kv.shape[0] == 2 and q.shape[0] == kv.shape[1]
    _out = None
    _lse = None
    for ring_idx in range(WORLD):
        _q = q[:, :, :, :]
        if ring_idx == 0:
            _kv = kv[:, :, :, :, :].contiguous()
            comm = SendRecv()
        else:
            comm.wait()
            _kv = _next_kv
        if ring_idx + 1 != WORLD:
            send_to = n_dim_to_one_dim(shift_tuple_element(indices, 0, 1, WORLD), (WORLD,))
            recv_from = n_dim_to_one_dim(shift_tuple_element(indices, 0, -1, WORLD), (WORLD,))
            _next_kv = comm.send_recv(send_to, recv_from, _kv)
            comm.commit()
        _k = _kv[0]
        _v = _kv[1]
        params = get_default_args(_flash_attn_forward).copy()
        params.update({"q": _q, "k": _k, "v": _v, "dropout_p": dropout_p, "softmax_scale": softmax_scale,
                       "causal": causal, "alibi_slopes": alibi_slopes, "return_softmax": True and dropout_p > 0,
                       "window_size_left": window_size[0], "window_size_right": window_size[1]})
        outputs = _flash_attn_forward(**params)
        assert len(outputs) == 4
        block_out, block_lse, _, _ = outputs
        _out, _lse = update_out_and_lse(_out, _lse, block_out, block_lse)
    o[:, :, :, :] = _out.to(q.dtype)
    lse[:, :, :] = _lse.squeeze(dim=-1).transpose(1, 2)
'''

PACKED_REDUCE_TEXT = '''
def ring_step_packed(q, kv, o, lse, softmax_scale, dropout_p=0, causal=False, window_size=(-1, -1),
                     alibi_slopes=None, deterministic=False):
    indices = one_dim_to_n_dim(dist.get_rank(), (WORLD,))
    buf = None
    for ring_idx in range(WORLD):
        if ring_idx == 0:
            _kv = kv[:, :, :, :, :].contiguous()
            comm = SendRecv()
        else:
            comm.wait()
            _kv = _next_kv
        if ring_idx + 1 != WORLD:
            send_to = n_dim_to_one_dim(shift_tuple_element(indices, 0, 1, WORLD), (WORLD,))
            recv_from = n_dim_to_one_dim(shift_tuple_element(indices, 0, -1, WORLD), (WORLD,))
            _next_kv = comm.send_recv(send_to, recv_from, _kv)
            comm.commit()
        params = get_default_args(_flash_attn_forward).copy()
        params.update({"q": q, "k": _kv[0], "v": _kv[1], "dropout_p": dropout_p, "softmax_scale": softmax_scale,
                       "causal": causal, "alibi_slopes": alibi_slopes, "return_softmax": True and dropout_p > 0,
                       "window_size_left": window_size[0], "window_size_right": window_size[1]})
        outputs = _flash_attn_forward(**params)
        block_out, block_lse, _, _ = outputs
        src = torch.cat([block_out.to(torch.float32), block_lse.transpose(-2, -1).unsqueeze(dim=-1)], dim=-1)
        buf = src if buf is None else flash_reduce(buf, src)
    o[:, :, :, :] = buf[..., :-1].to(q.dtype)
    lse[:, :, :] = buf[..., -1].transpose(1, 2)
'''

BACKWARD_TEXT = '''
def ring_step_backward(q, kv, o, lse, dout, dq, dkv, softmax_scale, dropout_p=0, causal=False,
                       window_size=(-1, -1), alibi_slopes=None, deterministic=False):
    indices = one_dim_to_n_dim(dist.get_rank(), (WORLD,))
    reduce_dq = None
    for ring_idx in range(WORLD):
        if ring_idx == 0:
            _kv = kv[:, :, :, :, :].contiguous()
            comm = SendRecv()
        else:
            comm.wait()
            _kv = _next_kv
        if ring_idx + 1 != WORLD:
            send_to = n_dim_to_one_dim(shift_tuple_element(indices, 0, 1, WORLD), (WORLD,))
            recv_from = n_dim_to_one_dim(shift_tuple_element(indices, 0, -1, WORLD), (WORLD,))
            _next_kv = comm.send_recv(send_to, recv_from, _kv)
            comm.commit()
        block_dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        block_dkv = torch.empty(_kv.shape, dtype=kv.dtype, device=kv.device)
        params = get_default_args(_flash_attn_backward).copy()
        params.update({"dout": dout, "q": q, "k": _kv[0], "v": _kv[1], "out": o, "softmax_lse": lse,
                       "dq": block_dq, "dk": block_dkv[0], "dv": block_dkv[1], "softmax_scale": softmax_scale,
                       "dropout_p": dropout_p, "causal": False, "deterministic": deterministic,
                       "alibi_slopes": alibi_slopes})
        if "window_size" in params:
            params.update({"window_size": window_size})
        else:
            params.update({"window_size_left": window_size[0], "window_size_right": window_size[1]})
        _flash_attn_backward(**params)
        if reduce_dq is None:
            reduce_dq = block_dq.to(torch.float32)
        else:
            reduce_dq = torch.add(reduce_dq, block_dq.to(torch.float32))
        if ring_idx == 0:
            dkv[...] = block_dkv
    dq[...] = reduce_dq.to(dq.dtype)
'''


class _Dist:
    def __init__(self, rank):
        self._rank = rank

    def get_rank(self):
        return self._rank


@pytest.mark.parametrize("text,name", [(SINGLE_RING_TEXT, "ring_step"), (PACKED_REDUCE_TEXT, "ring_step_packed")])
@pytest.mark.parametrize("rank", [0, 2])
def test_generated_style_text_runs_in_the_namespace(text, name, rank):
    import mercury_artifact_amd as M

    B, S, H, D, W = 2, 1024, 3, 128, 4
    g = torch.Generator().manual_seed(21)
    q = torch.randn(B, S // W, H, D, generator=g).bfloat16()
    kvs = [torch.randn(2, B, S // W, H, D, generator=g).bfloat16() for _ in range(W)]
    scale = D ** -0.5
    ro, rl = O.ring_forward(q.float(), [c.float() for c in kvs], O.single_ring_order(rank, W), scale)
    dev = [c.cuda() for c in kvs]
    ring = M.LocalRing((W,), rank, dev)
    namespace = {"torch": torch, "os": os, "dist": _Dist(rank), "WORLD": W, "SendRecv": lambda: ring}
    namespace.update(M.namespace(lazy_merge=False))
    exec(text, namespace)
    o = torch.empty(B, S // W, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
    namespace[name](q.cuda(), dev[rank], o, lse, scale)
    torch.cuda.synchronize()
    assert (o.float().cpu() - ro).abs().max().item() <= 2e-2
    assert ((lse.cpu() - rl).abs() / rl.abs().clamp_min(1.0)).max().item() <= 1e-3
    # and it is what the package's own driver gives, bit for bit, when that runs the literal sequence
    if name == "ring_step":
        o2, lse2 = torch.empty_like(o), torch.empty_like(lse)
        M.flash_attn_pack_kv(q.cuda(), dev[rank], o2, lse2, scale, ring=M.LocalRing((W,), rank, dev),
                             deferred_merge=False, fused_epilogue=False)
        assert torch.equal(o, o2) and torch.equal(lse, lse2)


ZIGZAG_STYLE_TEXT = '''
def two_block_step(q, kv_a, kv_b, o, lse, softmax_scale):
    half = q.shape[1] // 2
    _out = None
    _lse = None
    for idx, (_q, _kv, sl) in enumerate([(q, kv_a, None), (q[:, half:], kv_b, (slice(None), slice(half, None)))]):
        params = get_default_args(_flash_attn_forward).copy()
        params.update({"q": _q, "k": _kv[0], "v": _kv[1], "dropout_p": 0, "softmax_scale": softmax_scale,
                       "causal": False, "alibi_slopes": None, "return_softmax": False,
                       "window_size_left": -1, "window_size_right": -1})
        block_out, block_lse, _, _ = _flash_attn_forward(**params)
        _out, _lse = update_out_and_lse(_out, _lse, block_out, block_lse, slice_=sl)
    o[:, :, :, :] = _out.to(q.dtype)
    lse[:, :, :] = _lse.squeeze(dim=-1).transpose(1, 2)
'''


@pytest.mark.parametrize("rank", [0, 3])
def test_unchanged_text_in_the_lazy_namespace_folds_once(rank):
    """SINGLE_RING_TEXT, not a character changed, exec-ed in namespace(lazy_merge=True): update_out_and_lse only
    records, the epilogue expressions trigger ONE merge_many call and no merge_into call; the result passes the
    oracle gates and agrees with the literal chain to fp32 rounding of the accumulator (one bf16 ulp on out)."""
    import mercury_artifact_amd as M
    from mercury_artifact_amd import lazy as L
    from mercury_artifact_amd import merge as MG

    B, S, H, D, W = 2, 1024, 3, 128, 4
    g = torch.Generator().manual_seed(21)
    q = torch.randn(B, S // W, H, D, generator=g).bfloat16()
    kvs = [torch.randn(2, B, S // W, H, D, generator=g).bfloat16() for _ in range(W)]
    scale = D ** -0.5
    ro, rl = O.ring_forward(q.float(), [c.float() for c in kvs], O.single_ring_order(rank, W), scale)
    dev = [c.cuda() for c in kvs]
    results = {}
    calls = {"many": 0, "into": 0}
    real_many, real_into = MG.merge_many, MG.merge_into

    def count_many(*a, **kw):
        calls["many"] += 1
        return real_many(*a, **kw)

    def count_into(*a, **kw):
        calls["into"] += 1
        return real_into(*a, **kw)

    for lazy in (False, True):
        ring = M.LocalRing((W,), rank, dev)
        namespace = {"torch": torch, "os": os, "dist": _Dist(rank), "WORLD": W, "SendRecv": lambda: ring}
        namespace.update(M.namespace(lazy_merge=lazy))
        exec(SINGLE_RING_TEXT, namespace)
        o = torch.empty(B, S // W, H, D, dtype=torch.bfloat16, device="cuda")
        lse = torch.empty(B, H, S // W, dtype=torch.float32, device="cuda")
        calls.update(many=0, into=0)
        MG.merge_many, MG.merge_into = count_many, count_into
        try:
            namespace["ring_step"](q.cuda(), dev[rank], o, lse, scale)
        finally:
            MG.merge_many, MG.merge_into = real_many, real_into
        torch.cuda.synchronize()
        assert (calls["many"], calls["into"]) == ((1, 0) if lazy else (0, W))
        assert (o.float().cpu() - ro).abs().max().item() <= 2e-2
        assert ((lse.cpu() - rl).abs() / rl.abs().clamp_min(1.0)).max().item() <= 1e-3
        results[lazy] = (o.float().cpu(), lse.cpu())
    d_out = (results[True][0] - results[False][0]).abs()
    assert (d_out - 2 ** -7 * results[False][0].abs()).max().item() <= 1e-6      # at most one bf16 ulp apart
    assert (results[True][1] - results[False][1]).abs().max().item() <= 1e-5


def test_lazy_handles_fall_back_to_the_literal_chain():
    """Whatever is done to the handles beyond the generated epilogue gives what real accumulators give: a slice_
    merge on a row range (recorded, folded), a torch function and an attribute on a handle (chain), a functional
    call that leaves the earlier handles valid, and the first-call error."""
    import mercury_artifact_amd as M
    from mercury_artifact_amd import lazy as L

    B, Sq, H, D = 1, 256, 2, 128
    g = torch.Generator().manual_seed(23)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16().cuda()
    kva = torch.randn(2, B, 192, H, D, generator=g).bfloat16().cuda()
    kvb = torch.randn(2, B, 128, H, D, generator=g).bfloat16().cuda()
    scale = D ** -0.5
    outs = {}
    for lazy in (False, True):
        namespace = {"torch": torch}
        namespace.update(M.namespace(lazy_merge=lazy))
        exec(ZIGZAG_STYLE_TEXT, namespace)
        o = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
        lse = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
        namespace["two_block_step"](q, kva, kvb, o, lse, scale)
        outs[lazy] = (o.float().cpu(), lse.cpu())
    assert (outs[True][0] - outs[False][0]).abs().max().item() <= 2 ** -7 * outs[False][0].abs().max().item() + 1e-6
    assert (outs[True][1] - outs[False][1]).abs().max().item() <= 1e-5
    # handles used like tensors
    bo1, bl1 = M.attn_fwd_block(q, kva[0], kva[1], scale)
    bo2, bl2 = M.attn_fwd_block(q, kvb[0], kvb[1], scale)
    h_out, h_lse = L.update_out_and_lse_lazy(None, None, bo1, bl1)
    assert isinstance(h_out, L.LazyOut) and isinstance(h_lse, L.LazyLse)
    assert h_out.shape == (B, Sq, H, D) and h_lse.shape == (B, Sq, H, 1) and h_out.dtype == torch.float32
    h2_out, h2_lse = L.update_out_and_lse_lazy(h_out, h_lse, bo2, bl2)
    r_out, r_lse = M.update_out_and_lse(*M.update_out_and_lse(None, None, bo1, bl1), bo2, bl2)
    assert torch.equal(torch.add(h2_out, 0.0), r_out)                     # torch function -> literal chain
    assert torch.equal(h2_lse.float().squeeze(-1), r_lse.squeeze(-1))     # attribute -> literal chain
    assert torch.equal(h_out.to(torch.float32), bo1.float())              # the earlier handles still stand for one block
    assert torch.equal(h2_out.to(torch.bfloat16), r_out.to(torch.bfloat16))   # after the chain ran: its cast
    with pytest.raises(RuntimeError):
        L.update_out_and_lse_lazy(None, None, bo1, bl1, slice_=(slice(None), slice(0, 8)))
    # a slice_ the fold cannot express (a row range that stops early) is merged literally, in place
    h3_out, h3_lse = L.update_out_and_lse_lazy(None, None, bo1, bl1)
    same_out, same_lse = L.update_out_and_lse_lazy(h3_out, h3_lse, bo2[:, :64].contiguous(), bl2[:, :, :64].contiguous(),
                                                   slice_=(slice(None), slice(0, 64)))
    assert same_out is h3_out and same_lse is h3_lse
    e_out, e_lse = M.update_out_and_lse(None, None, bo1, bl1)
    M.update_out_and_lse(e_out, e_lse, bo2[:, :64].contiguous(), bl2[:, :, :64].contiguous(), slice_=(slice(None), slice(0, 64)))
    assert torch.equal(h3_out.to(torch.bfloat16), e_out.to(torch.bfloat16))
    assert torch.equal(h3_lse.squeeze(dim=-1).transpose(1, 2), e_lse.squeeze(dim=-1).transpose(1, 2))


def test_generated_style_backward_text():
    import mercury_artifact_amd as M

    B, S, H, D, W, rank = 1, 1024, 3, 128, 4, 1
    g = torch.Generator().manual_seed(22)
    q = torch.randn(B, S // W, H, D, generator=g).bfloat16()
    kvs = [torch.randn(2, B, S // W, H, D, generator=g).bfloat16() for _ in range(W)]
    dout = torch.randn(B, S // W, H, D, generator=g).bfloat16()
    scale = D ** -0.5
    order = O.single_ring_order(rank, W)
    o, lse = O.ring_forward(q.float(), [c.float() for c in kvs], order, scale)
    o16 = o.bfloat16()
    rdq, rdkv = O.ring_backward(q.float(), [c.float() for c in kvs], order, o16.float(), lse, dout.float(), scale)
    dev = [c.cuda() for c in kvs]
    ring = M.LocalRing((W,), rank, dev)
    namespace = {"torch": torch, "os": os, "dist": _Dist(rank), "WORLD": W, "SendRecv": lambda: ring}
    namespace.update(M.namespace())
    exec(BACKWARD_TEXT, namespace)
    dq = torch.empty_like(q, device="cuda")
    dkv = torch.empty_like(dev[rank])
    namespace["ring_step_backward"](q.cuda(), dev[rank], o16.cuda(), lse.cuda(), dout.cuda(), dq, dkv, scale)
    torch.cuda.synchronize()

    def rel(a, b):
        return (a.float().cpu() - b).norm().item() / b.norm().item()

    assert rel(dq, rdq) <= 1e-2
    assert rel(dkv[0], rdkv[rank][0]) <= 1e-2 and rel(dkv[1], rdkv[rank][1]) <= 1e-2
