#!/usr/bin/env python3
"""Writes tests/golden/schedules_and_e4m3.json: known answers worked out from first principles, without the
oracle and without this package, for the integer parts of the ring step.

  * chunk orders: every rank of the mesh holds the chunk with its own number, and in every step every rank
    hands what it holds to its +1 neighbour along one mesh dimension (dimension 0 unless the inner loop is
    at its last step, then the next dimension) -- simulated by moving list entries around;
  * zigzag step classes: rank r of W holds sequence blocks r and 2W-1-r; a (query block, key block) pair is
    visible iff the key block is not after the query block, which fixes what part of every chunk a rank
    needs at every step;
  * the value of every OCP e4m3fn code from its bit layout (1 sign, 4 exponent bits with bias 7, 3 mantissa
    bits; exponent 0 is subnormal; 0x7f / 0xff are NaN; there is no infinity).

The reference's tests hold no golden vector for this path (they compare two flash-attn results on unseeded
data), and nothing of the reference was imported to make these.
"""
import json
import os


def simulate_orders(mesh):
    """order[rank] = chunk ids in the order the rank holds them; mesh dimension 0 is the fastest digit."""
    world = 1
    for m in mesh:
        world *= m
    holds = list(range(world))                    # holds[rank] = chunk id
    order = [[] for _ in range(world)]

    def coords(rank):
        c = []
        for m in mesh:
            c.append(rank % m)
            rank //= m
        return c

    def rank_of(c):
        r, mul = 0, 1
        for x, m in zip(c, mesh):
            r += x * mul
            mul *= m
        return r

    counters = [0] * len(mesh)
    for _ in range(world):
        for r in range(world):
            order[r].append(holds[r])
        # which dimension hops: the first one whose loop is not at its last step
        dim = None
        for d in range(len(mesh)):
            if counters[d] + 1 != mesh[d]:
                dim = d
                break
        if dim is not None:
            new = [None] * world
            for r in range(world):
                c = coords(r)
                c[dim] = (c[dim] + 1) % mesh[dim]
                new[rank_of(c)] = holds[r]
            holds = new
        for d in range(len(mesh)):
            counters[d] += 1
            if counters[d] < mesh[d]:
                break
            counters[d] = 0
    return order


def zigzag_classes(world):
    """classes[rank][step] for the single ring order: what the rank needs of the chunk it holds at that step."""
    out = []
    for r in range(world):
        q_blocks = (r, 2 * world - 1 - r)
        row = []
        for step in range(world):
            src = (r - step) % world
            k_blocks = (src, 2 * world - 1 - src)
            vis = [[kb <= qb for kb in k_blocks] for qb in q_blocks]   # [query half][key half], block granularity
            if src == r:
                row.append("diag")
            elif vis == [[True, False], [True, False]]:
                row.append("kv_first_half")
            elif vis == [[False, False], [True, True]]:
                row.append("q_second_half")
            else:
                raise AssertionError((r, step, vis))
        out.append(row)
    return out


def e4m3_value(code):
    sign = -1.0 if code & 0x80 else 1.0
    e, m = (code >> 3) & 0xF, code & 7
    if e == 15 and m == 7:
        return None                                # NaN
    if e == 0:
        return sign * (m / 8.0) * 2.0 ** -6
    return sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)


def main():
    data = {
        "orders": {"x".join(map(str, mesh)): simulate_orders(mesh)
                   for mesh in ([4], [8], [2, 2], [4, 2], [2, 4], [2, 2, 2])},
        "zigzag": {str(w): zigzag_classes(w) for w in (2, 4, 8)},
        "e4m3": [e4m3_value(c) for c in range(256)],
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "schedules_and_e4m3.json")
    with open(path, "w") as f:
        json.dump(data, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
