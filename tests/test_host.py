"""CPU-only checks of the host side: the C-ABI library loads and exports every symbol the header
declares, the operators expose the keyword surface the generated code relies on, the product's
schedule helpers agree with the oracle's (which is pinned by simulation), and the operators refuse
to run without a GPU instead of falling back."""
import ctypes
import os
import re

import pytest
import torch

import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from mercury_artifact_amd import _native

    header = open(os.path.join(ROOT, "include", "mercury_hip.h")).read()
    declared = set(re.findall(r"\b(mhip_[a-z0-9_]+)\s*\(", header))
    assert declared and declared == set(_native.EXPORTED_SYMBOLS)
    handle = ctypes.CDLL(_native.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name
    lib = _native.lib()
    assert lib.mhip_version() >= 1
    assert lib.mhip_error_string(0) == b"ok" and b"head dimension" in lib.mhip_error_string(-3)


def test_keyword_surface_of_the_block_operators():
    import mercury_artifact_amd as M

    fwd = M.get_default_args(M._flash_attn_forward)
    for key in ("q", "k", "v", "dropout_p", "softmax_scale", "causal", "window_size_left",
                "window_size_right", "softcap", "alibi_slopes", "return_softmax"):
        assert key in fwd
    assert list(fwd)[:11] == ["q", "k", "v", "dropout_p", "softmax_scale", "causal", "window_size_left",
                              "window_size_right", "softcap", "alibi_slopes", "return_softmax"]
    assert fwd["softcap"] == 0.0 and fwd["q"] is None and fwd["q_descale"] is None
    bwd = M.get_default_args(M._flash_attn_backward)
    for key in ("dout", "q", "k", "v", "out", "softmax_lse", "dq", "dk", "dv", "softmax_scale",
                "dropout_p", "causal", "deterministic", "alibi_slopes", "window_size_left",
                "window_size_right", "softcap", "rng_state"):
        assert key in bwd
    # plain functions work too, and the cached dict must be copied by callers
    def f(a, b=2, softcap=5.0):
        return a
    assert M.get_default_args(f) == {"a": None, "b": 2, "softcap": 0.0}
    ns = M.namespace()
    for name in ("_flash_attn_forward", "_flash_attn_backward", "get_default_args", "update_out_and_lse",
                 "flash_reduce", "one_dim_to_n_dim", "n_dim_to_one_dim", "shift_tuple_element",
                 "get_src_dst_ranks"):
        assert callable(ns[name])


def test_no_cpu_fallback():
    import mercury_artifact_amd as M

    q = torch.randn(1, 8, 1, 128).bfloat16()
    with pytest.raises(RuntimeError):
        M.attn_fwd_block(q, q, q, 0.1)
    with pytest.raises((RuntimeError, NotImplementedError)):
        M._flash_attn_forward(q=q, k=q, v=q, dropout_p=0, softmax_scale=0.1, causal=False,
                              window_size_left=-1, window_size_right=-1, softcap=0.0,
                              alibi_slopes=None, return_softmax=False)
    with pytest.raises(RuntimeError):
        M.update_out_and_lse(None, None, q, torch.zeros(1, 1, 8))
    with pytest.raises(RuntimeError):
        M.flash_reduce(torch.zeros(4, 129), torch.zeros(4, 129))
    with pytest.raises(RuntimeError):
        M.update_out_and_lse(None, None, q, torch.zeros(1, 1, 8), slice_=(slice(None),))


def test_index_helpers():
    import mercury_artifact_amd as M

    for shape in [(8,), (4, 2), (2, 2, 2), (3, 5)]:
        world = 1
        for s in shape:
            world *= s
        seen = set()
        for r in range(world):
            idx = M.one_dim_to_n_dim(r, shape)
            assert idx[0] == r % shape[0]                     # dimension 0 is the fastest digit
            assert M.n_dim_to_one_dim(idx, shape) == r
            seen.add(idx)
        assert len(seen) == world
    assert M.shift_tuple_element((0, 1), 0, -1, 4) == (3, 1)
    assert M.shift_tuple_element((3, 1), 0, 1, 4) == (0, 1)
    # single ring: source is rank-1, destination rank+1
    assert M.get_src_dst_ranks((2,), (8,), [0]) == (1, 3)
    # double ring (4, 2), ring dims [1, 0]: dim 0 shifts by 1, then dim 1 by the size of dim 0 (mod 2 -> 0)
    assert M.get_src_dst_ranks((0, 0), (4, 2), [1, 0]) == (3, 1)


@pytest.mark.parametrize("world", [1, 2, 4, 8])
def test_product_schedules_equal_oracle(world):
    import mercury_artifact_amd as M

    for r in range(world):
        assert M.single_ring_order(r, world) == O.single_ring_order(r, world)
        for step in range(world):
            assert M.zigzag_step(r, step, world) == O.zigzag_step(r, step, world)
        assert M.zigzag_blocks(r, world) == O.zigzag_blocks(r, world)
    assert M.ring_divide_order(world - 1, world, 2) == O.ring_divide_order(world - 1, world, 2)


@pytest.mark.parametrize("inner,outer", [(4, 2), (2, 2), (2, 4), (1, 3), (3, 1)])
def test_product_double_ring_equals_oracle(inner, outer):
    import mercury_artifact_amd as M

    for r in range(inner * outer):
        assert M.double_ring_order(r, inner, outer) == O.double_ring_order(r, inner, outer)


def test_local_ring_protocol_errors():
    import mercury_artifact_amd as M

    chunks = [torch.full((1,), float(i)) for i in range(4)]
    ring = M.LocalRing((4,), 1, chunks)
    with pytest.raises(RuntimeError):
        ring.wait()                                   # wait before commit
    got = ring.send_recv(2, 0, chunks[1])
    assert got.item() == 0.0                          # rank 1 receives rank 0's chunk
    ring.commit()
    with pytest.raises(RuntimeError):
        ring.commit()                                 # commit twice
    ring.wait()
    with pytest.raises(RuntimeError):
        ring.send_recv(3, 0, chunks[1])               # not a +1 / -1 hop
    with pytest.raises(ValueError):
        M.LocalRing((4,), 7)
    with pytest.raises(ValueError):
        M.LocalRing((4,), 0, chunks[:2])


def test_quantize_e4m3_has_no_cpu_path():
    import mercury_artifact_amd as M

    with pytest.raises(RuntimeError):
        M.quantize_e4m3(torch.randn(1000))


@pytest.mark.parametrize("mesh", [(4,), (8,), (4, 2), (2, 3), (2, 2, 2)])
def test_reduce_buffer_route_visits_every_rank_once_and_returns_home(mesh):
    """Follow every ringed reduce buffer by hand: it must be at a different rank at every step (so it
    folds in every KV shard exactly once) and the write-back hop must land it on the rank it started on."""
    import mercury_artifact_amd as M

    sends, home = M.reduce_buffer_route(mesh)
    world = len(home)
    assert len(sends) == world - 1
    for start in range(world):
        at, seen = start, [start]
        for s in range(world - 1):
            at = sends[s][at]
            seen.append(at)
        assert sorted(seen) == list(range(world))
        assert home[at] == start
    for s in range(world - 1):
        assert sorted(sends[s]) == list(range(world))        # a hop is a permutation of the ranks


def test_get_device_group_is_the_reference_grouping():
    """Ranks whose coordinates agree outside `dims` (mercury/backend/pytorch/utils.py:114-169), by brute force over
    the mesh; debug=True gives the rank tuple, otherwise a LocalGroup over the same ranks."""
    import itertools

    import mercury_artifact_amd as M

    for mesh_shape in [(4,), (2, 2), (4, 2), (2, 3, 2)]:
        world = 1
        for m in mesh_shape:
            world *= m
        for k in range(1, len(mesh_shape) + 1):
            for dims in itertools.combinations(range(len(mesh_shape)), k):
                for rank in range(world):
                    idx = M.one_dim_to_n_dim(rank, mesh_shape)
                    want = tuple(r for r in range(world)
                                 if all(M.one_dim_to_n_dim(r, mesh_shape)[d] == idx[d]
                                        for d in range(len(mesh_shape)) if d not in dims))
                    assert M.get_device_group(idx, mesh_shape, dims, debug=True) == want
                    group = M.get_device_group(idx, mesh_shape, dims)
                    assert group.ranks == want and group.ranks[group.rank] == rank and group.size() == len(want)
    with pytest.raises(ValueError):
        M.get_device_group((0, 0), (2, 2), (2,))
    # on one GPU the other ranks' operands have to come from somewhere
    group = M.get_device_group((1,), (4,), (0,))
    with pytest.raises(RuntimeError):
        group.operands(torch.zeros(1))
    with M.local_peers(lambda r: torch.full((1,), float(r))):
        assert [t.item() for t in group.operands(torch.full((1,), -1.0))] == [0.0, -1.0, 2.0, 3.0]


def test_debug_print_prefixes_the_rank(capsys):
    import mercury_artifact_amd as M

    M.namespace()["debug_print"]("x", 3)
    assert capsys.readouterr().out == "[Rank 0] x 3\n"


def test_local_mesh_replays_the_ring_protocol_of_all_ranks():
    """Every rank as a thread: what arrives hop by hop is the chunk order of LocalRing / the oracle; SendRecv misuse
    raises as in the reference; a rank waiting for a message nobody sends raises instead of hanging."""
    import mercury_artifact_amd as M
    import oracle as O

    inner, outer = 4, 2
    mesh = M.LocalMesh((inner, outer))

    def rank_fn(r):
        indices = M.one_dim_to_n_dim(mesh.dist.get_rank(), (inner, outer))
        seen = []
        for o in range(outer):
            for i in range(inner):
                if i == 0 and o == 0:
                    cur = torch.tensor([float(r)])
                    comm = mesh.SendRecv()
                else:
                    comm.wait()
                    cur = nxt
                seen.append(int(cur.item()))
                if i + 1 != inner:
                    to = M.n_dim_to_one_dim(M.shift_tuple_element(indices, 0, 1, inner), (inner, outer))
                    frm = M.n_dim_to_one_dim(M.shift_tuple_element(indices, 0, -1, inner), (inner, outer))
                    nxt = comm.send_recv(to, frm, cur)
                    comm.commit()
                elif o + 1 != outer:
                    to = M.n_dim_to_one_dim(M.shift_tuple_element(indices, 1, 1, outer), (inner, outer))
                    frm = M.n_dim_to_one_dim(M.shift_tuple_element(indices, 1, -1, outer), (inner, outer))
                    nxt = comm.send_recv(to, frm, cur)
                    comm.commit()
        return seen

    orders = mesh.run(rank_fn)
    for r in range(inner * outer):
        assert orders[r] == O.double_ring_order(r, inner, outer) == M.double_ring_order(r, inner, outer)

    small = M.LocalMesh((2,), timeout=0.5)

    def misuse(r):
        comm = small.SendRecv()
        with pytest.raises(RuntimeError, match="wait called before commit"):
            comm.wait()
        comm.send_recv(1 - r, 1 - r, torch.zeros(1))
        comm.commit()
        with pytest.raises(RuntimeError, match="commit called twice"):
            comm.commit()
        comm.wait()
        return small.dist.get_world_size()

    assert small.run(misuse) == [2, 2]

    def starved(r):
        comm = small.SendRecv()
        if r == 0:
            comm.send_recv(1, 1, torch.zeros(1))
            comm.commit()
            comm.wait()

    with pytest.raises(RuntimeError, match="waited"):
        small.run(starved)


def test_local_mesh_reports_the_first_failure_and_releases_the_waiting_ranks():
    """A rank that raises ends the whole run at once: the ranks waiting for its messages stop waiting (they do not sit
    out the time limit), and what run() raises is that rank's own exception, whichever rank index it had."""
    import time

    import mercury_artifact_amd as M

    mesh = M.LocalMesh((4,), timeout=30.0)

    def rank_fn(r):
        comm = mesh.SendRecv()
        if r == 3:
            time.sleep(0.2)                      # the others are waiting by now
            raise ValueError("rank 3 broke")
        comm.send_recv((r + 1) % 4, (r - 1) % 4, torch.zeros(1))
        comm.commit()
        comm.wait()                              # rank 0 waits for rank 3, which never sends
        return r

    begin = time.monotonic()
    with pytest.raises(ValueError, match="rank 3 broke"):
        mesh.run(rank_fn)
    assert time.monotonic() - begin < 5.0
    # the mesh is usable again afterwards: the messages of the failed run are gone, the barrier works
    def again(r):
        comm = mesh.SendRecv()
        got = comm.send_recv((r + 1) % 4, (r - 1) % 4, torch.full((1,), float(r + 10)))
        comm.commit()
        comm.wait()
        mesh.dist.barrier()
        return int(got.item())

    assert mesh.run(again) == [13, 10, 11, 12]
