"""The text Mercury's own generator emits (tests/golden/generated_steps.json, written by
tests/golden/make_generated_steps.py from the reference's templates and schedule calls) exec-ed against this
package: every rank of the mesh at once through ``LocalMesh``, every rank's result against the CPU oracle.

The function text is run as generated.  Only the four import lines above it are left out: they set up the
reference's environment (``import torch.distributed as dist``, ``from mercury.backend import *``), which here is
the dict the text is exec-ed in -- ``dist`` and ``SendRecv`` of the mesh stand-in and ``namespace()`` of this
package.

Layout of the inputs: a tensor that a recipe shards over mesh dimensions ``dims`` is cut into as many equal row
blocks as those dimensions have ranks, and a rank holds the block numbered by its coordinates on them (first
listed dimension fastest); every rank must end with attention of ITS query rows over ALL keys, whatever the
schedule in between (ring, double ring, sub-chunk loops, tree collective, travelling reduce buffer).
"""
import json
import os

import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "generated_steps.json")) as _fh:
    RECIPES = json.load(_fh)["recipes"]
FORWARD = [r for r in RECIPES if not r["name"].startswith("backward")]
BACKWARD = [r for r in RECIPES if r["name"].startswith("backward")]


def _function_text(code):
    head, body = code.split("\ndef ", 1)
    assert [l for l in head.splitlines() if l.strip()] == ["import os", "import torch", "import torch.distributed as dist",
                                                          "from mercury.backend import *"]
    return "def " + body


def _shard(rank, mesh, dims):
    """(index, count) of the block a rank holds of a tensor sharded over mesh dimensions ``dims``."""
    import mercury_artifact_amd as M

    coords = M.one_dim_to_n_dim(rank, tuple(mesh))
    index, count = 0, 1
    for d in dims:
        index += coords[d] * count
        count *= mesh[d]
    return index, count


def _namespace(M, mesh, lazy):
    os.environ.setdefault("LOCAL_RANK", "0")
    ns = {"torch": torch, "os": os, "dist": mesh.dist, "SendRecv": mesh.SendRecv}
    ns.update(M.namespace(lazy_merge=lazy))
    return ns


def test_the_fixture_covers_the_schedules_of_the_reference():
    names = {r["name"] for r in RECIPES}
    assert {"single_ring_divide_1", "single_ring_divide_4", "double_ring_2x2", "gqa_single_ring", "tree_attention",
            "reduce_ring", "double_reduce_ring_2x2", "tree_over_ring_2x2", "backward_kv_ring", "backward_q_ring",
            "backward_kv_sharded_collective", "backward_q_sharded_collective"} <= names
    text = "\n".join(r["code"] for r in RECIPES)
    for needle in ("update_out_and_lse_collective(reduce_buf, dist.all_reduce, group=get_device_group(indices,",
                   "add_collective(", "get_src_dst_ranks(indices, (2, 2), [0, 1])", "flash_reduce(_next_reduce_buf, block_res)",
                   "elif S_kv_outer_ring_idx + 1 != 2:", "get_default_args(_flash_attn_backward).copy()"):
        assert needle in text, needle


@pytest.mark.parametrize("lazy", [True, False])
@pytest.mark.parametrize("recipe", FORWARD, ids=[r["name"] for r in FORWARD])
def test_generated_forward_step_of_every_rank_matches_the_oracle(recipe, lazy):
    import mercury_artifact_amd as M

    mesh_shape = tuple(recipe["mesh"])
    B, S, Hq, Hkv, D = (recipe[k] for k in ("B", "S", "Hq", "Hkv", "D"))
    scale = D ** -0.5
    g = torch.Generator().manual_seed(41)
    q = torch.randn(B, S, Hq, D, generator=g).bfloat16()
    kv = torch.randn(2, B, S, Hkv, D, generator=g).bfloat16()
    mesh = M.LocalMesh(mesh_shape)
    ns = _namespace(M, mesh, lazy)
    exec(_function_text(recipe["code"]), ns)
    func = ns[recipe["function"]]
    qd, kvd = q.cuda(), kv.cuda()
    outs = {}

    def rank_fn(rank):
        qi, qn = _shard(rank, mesh_shape, recipe["q_dims"])
        ki, kn = _shard(rank, mesh_shape, recipe["kv_dims"])
        q_loc = qd.chunk(qn, dim=1)[qi].contiguous()
        kv_loc = kvd.chunk(kn, dim=2)[ki].contiguous()
        o = torch.zeros_like(q_loc)
        lse = torch.zeros(B, Hq, q_loc.shape[1], dtype=torch.float32, device="cuda")
        func(q_loc, kv_loc, o, lse, scale, dropout_p=0, causal=False, window_size=(-1, -1), alibi_slopes=None,
             deterministic=False)
        outs[rank] = (qi, qn, o, lse)

    mesh.run(rank_fn)
    torch.cuda.synchronize()
    ro, rl = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale)
    for rank, (qi, qn, o, lse) in outs.items():
        want_o, want_l = ro.chunk(qn, dim=1)[qi], rl.chunk(qn, dim=2)[qi]
        assert (o.float().cpu() - want_o).abs().max().item() <= 2e-2, rank
        assert ((lse.cpu() - want_l).abs() / want_l.abs().clamp_min(1.0)).max().item() <= 1e-3, rank


@pytest.mark.parametrize("recipe", BACKWARD, ids=[r["name"] for r in BACKWARD])
def test_generated_backward_step_of_every_rank_matches_the_oracle(recipe):
    import mercury_artifact_amd as M

    mesh_shape = tuple(recipe["mesh"])
    B, S, H, D = (recipe[k] for k in ("B", "S", "Hq", "D"))
    scale = D ** -0.5
    g = torch.Generator().manual_seed(42)
    q = torch.randn(B, S, H, D, generator=g).bfloat16()
    kv = torch.randn(2, B, S, H, D, generator=g).bfloat16()
    dout = torch.randn(B, S, H, D, generator=g).bfloat16()
    o, lse = O.block_attention(q.float(), kv[0].float(), kv[1].float(), scale)
    o16 = o.bfloat16()
    rdq, rdk, rdv = O.block_backward(dout.float(), q.float(), kv[0].float(), kv[1].float(), o16.float(), lse, scale)
    mesh = M.LocalMesh(mesh_shape)
    ns = _namespace(M, mesh, True)
    exec(_function_text(recipe["code"]), ns)
    func = ns[recipe["function"]]
    dev = {name: t.cuda() for name, t in (("q", q), ("kv", kv), ("o", o16), ("lse", lse), ("dout", dout))}
    res = {}

    def rank_fn(rank):
        qi, qn = _shard(rank, mesh_shape, recipe["q_dims"])
        ki, kn = _shard(rank, mesh_shape, recipe["kv_dims"])
        rows = lambda t, dim: t.chunk(qn, dim=dim)[qi].contiguous()
        q_loc, o_loc, dout_loc = rows(dev["q"], 1), rows(dev["o"], 1), rows(dev["dout"], 1)
        lse_loc = rows(dev["lse"], 2)
        kv_loc = dev["kv"].chunk(kn, dim=2)[ki].contiguous()
        dq = torch.zeros_like(q_loc)
        dkv = torch.zeros_like(kv_loc)
        func(q_loc, kv_loc, o_loc, lse_loc, dout_loc, dq, dkv, scale, dropout_p=0, causal=False, window_size=(-1, -1),
             alibi_slopes=None, deterministic=False)
        res[rank] = (qi, qn, ki, kn, dq, dkv)

    mesh.run(rank_fn)
    torch.cuda.synchronize()

    def rel(a, b):
        return (a.float().cpu() - b).norm().item() / b.norm().item()

    for rank, (qi, qn, ki, kn, dq, dkv) in res.items():
        assert rel(dq, rdq.chunk(qn, dim=1)[qi]) <= 1e-2, rank
        assert rel(dkv[0], rdk.chunk(kn, dim=1)[ki]) <= 1e-2, rank
        assert rel(dkv[1], rdv.chunk(kn, dim=1)[ki]) <= 1e-2, rank


@pytest.mark.parametrize("name", ["single_ring_divide_2", "backward_kv_ring"])
def test_bench_program_allocates_from_the_reference_buffer_table_and_times_every_rank(name):
    """The search's timing harness (mercury/search/bench.py:15-86) on the reference's own lowering results: the text
    and the I/O buffer table of the fixture stand in for the four lowering calls, every rank of the mesh runs
    ``bench_program`` (zeros for written buffers, N(0,1) for the others, warm-up and timed calls), and what the timed
    function left in each rank's output buffers is the oracle's result on the tensors the harness allocated."""
    import threading
    import types

    import mercury_artifact_amd as M
    from mercury_artifact_amd import search_harness as SH

    recipe = next(r for r in RECIPES if r["name"] == name)
    W, D = recipe["mesh"][0], recipe["D"]
    scale = D ** -0.5
    mesh = M.LocalMesh(tuple(recipe["mesh"]))
    buffers = [types.SimpleNamespace(tensor=b["tensor"], shape=tuple(b["shape"]), dtype=getattr(torch, b["dtype"]),
                                     write=b["write"]) for b in recipe["io_buffers"]]
    low = SH.Lowering(eliminate_loops=lambda prog: None, generate_code=lambda prog: _function_text(recipe["code"]),
                      io_buffers=lambda prog: buffers, buffer_bytes=lambda prog: recipe["buffer_bytes"])
    os.environ.setdefault("LOCAL_RANK", "0")
    calls, timings = {}, {}
    real_bench_callable = SH.bench_callable

    def spy(func, call, *a, **kw):                   # the tensors the harness allocated, per rank thread
        calls[threading.get_ident()] = call
        return real_bench_callable(func, call, *a, **kw)

    def rank_fn(rank):
        extra = {"torch": torch, "os": os, "dist": mesh.dist, "SendRecv": mesh.SendRecv}
        timings[rank] = SH.bench_program(types.SimpleNamespace(name=recipe["function"]), extra, num_iter=2,
                                         kwargs={"softmax_scale": scale}, log=False, lowering=low)
        calls[rank] = calls.pop(threading.get_ident())

    SH.bench_callable = spy
    try:
        mesh.run(rank_fn)
    finally:
        SH.bench_callable = real_bench_callable
    torch.cuda.synchronize()
    assert sorted(calls) == list(range(W))
    for rank in range(W):
        ips, seconds, mem = timings[rank]
        assert ips > 0 and seconds > 0 and mem == recipe["buffer_bytes"]
        for b in buffers:
            t = calls[rank][b.tensor]
            assert tuple(t.shape) == b.shape and t.dtype == b.dtype and t.is_cuda

    def whole(tensor, dim):                          # the ranks' shards as one sequence
        return torch.cat([calls[r][tensor].float().cpu() for r in range(W)], dim=dim)

    q, kv = whole("q", 1), whole("kv", 2)
    if name.startswith("backward"):
        rdq, rdk, rdv = O.block_backward(whole("dout", 1), q, kv[0], kv[1], whole("o", 1), whole("lse", 2), scale)
        for rank in range(W):
            dq, dkv = calls[rank]["dq"].float().cpu(), calls[rank]["dkv"].float().cpu()
            for got, want in ((dq, rdq.chunk(W, dim=1)[rank]), (dkv[0], rdk.chunk(W, dim=1)[rank]),
                              (dkv[1], rdv.chunk(W, dim=1)[rank])):
                assert (got - want).norm().item() / want.norm().item() <= 1e-2, rank
    else:
        ro, rl = O.block_attention(q, kv[0], kv[1], scale)
        for rank in range(W):
            want_o, want_l = ro.chunk(W, dim=1)[rank], rl.chunk(W, dim=2)[rank]
            assert (calls[rank]["o"].float().cpu() - want_o).abs().max().item() <= 2e-2, rank
            assert ((calls[rank]["lse"].cpu() - want_l).abs() / want_l.abs().clamp_min(1.0)).max().item() <= 1e-3, rank
