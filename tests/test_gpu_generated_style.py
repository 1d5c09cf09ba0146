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
    namespace.update(M.namespace())
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
