"""The integer parts of the step against tests/golden/schedules_and_e4m3.json (known answers from a
message-passing simulation, from block visibility and from the e4m3 bit layout: tests/golden/make_fixtures.py).
Checked: the oracle, the package's schedule functions, and the hops LocalRing replays."""
import json
import math
import os

import pytest
import torch

import oracle as O
from mercury_artifact_amd import schedule as S

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_and_e4m3.json")) as f:
    GOLD = json.load(f)


@pytest.mark.parametrize("key", sorted(GOLD["orders"]))
def test_chunk_orders(key):
    mesh = tuple(int(x) for x in key.split("x"))
    orders = GOLD["orders"][key]
    world = len(orders)
    for rank in range(world):
        want = orders[rank]
        assert sorted(want) == list(range(world))                  # every chunk exactly once
        if len(mesh) == 1:
            assert O.single_ring_order(rank, world) == want
            assert S.single_ring_order(rank, world) == want
        if len(mesh) == 2:
            assert O.double_ring_order(rank, *mesh) == want
            assert S.double_ring_order(rank, *mesh) == want
        # the hops of the generated loop, replayed over local buffers
        chunks = [torch.full((1,), float(c)) for c in range(world)]
        ring = S.LocalRing(mesh, rank, chunks)
        seen = []
        counters = [0] * len(mesh)
        kv = chunks[rank]
        for step in range(world):
            seen.append(int(kv.item()))
            dim = next((d for d in range(len(mesh)) if counters[d] + 1 != mesh[d]), None)
            if dim is not None:
                me = S.one_dim_to_n_dim(rank, mesh)
                to = S.n_dim_to_one_dim(S.shift_tuple_element(me, dim, 1, mesh[dim]), mesh)
                frm = S.n_dim_to_one_dim(S.shift_tuple_element(me, dim, -1, mesh[dim]), mesh)
                nxt = ring.send_recv(to, frm, kv)
                ring.commit()
                ring.wait()
                kv = nxt
            for d in range(len(mesh)):
                counters[d] += 1
                if counters[d] < mesh[d]:
                    break
                counters[d] = 0
        assert seen == want
    if key == "4x2":
        assert orders[0] == [0, 3, 2, 1, 5, 4, 7, 6]


@pytest.mark.parametrize("world", sorted(int(w) for w in GOLD["zigzag"]))
def test_zigzag_step_classes(world):
    classes = GOLD["zigzag"][str(world)]
    for rank in range(world):
        for step in range(world):
            src = (rank - step) % world
            assert O.zigzag_step(rank, step, world) == (classes[rank][step], src)
            assert S.zigzag_step(rank, step, world) == (classes[rank][step], src)
        # equal work on every rank: one diagonal step, every other step half a block pair
        assert classes[rank].count("diag") == 1


def test_e4m3_code_table():
    table = GOLD["e4m3"]
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32)
    for c, want in enumerate(table):
        got = codes[c].item()
        if want is None:
            assert math.isnan(got)
        else:
            assert got == want, (c, got, want)
    finite = [v for v in table if v is not None]
    assert max(finite) == 448.0 and min(abs(v) for v in finite if v != 0) == 2.0 ** -9
    # the oracle's quantiser lands on table entries, and on the nearest one
    x = torch.linspace(-3, 3, 1001)
    xq, scale = O.quantize_e4m3(x)
    deq = O.dequantize(xq, scale)
    grid = torch.tensor(sorted(set(finite))) * scale
    nearest = grid[(x[:, None] - grid[None, :]).abs().argmin(dim=1)]
    assert ((deq - x).abs() <= (nearest - x).abs() + 1e-7).all()
