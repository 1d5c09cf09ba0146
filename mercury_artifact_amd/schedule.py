"""Rank <-> mesh index arithmetic and the local stand-in for the ring exchange.

The generated ring code gets these by ``from mercury.backend import *``
(mercury/backend/pytorch/utils.py:9-106,171-192).  On one GPU there is no peer to exchange with:
``LocalRing`` holds every rank's KV chunk, replays the hops all ranks would make together, and
hands the emulated rank the chunk it would have received -- buffer rotation in place of send/recv.
"""
from __future__ import annotations

from functools import lru_cache
from typing import List, Optional, Sequence, Tuple

import torch

__all__ = ["one_dim_to_n_dim", "n_dim_to_one_dim", "shift_tuple_element", "get_src_dst_ranks",
           "LocalRing", "single_ring_order", "double_ring_order", "ring_divide_order",
           "zigzag_blocks", "zigzag_step"]


@lru_cache(maxsize=None)
def one_dim_to_n_dim(one_dim_index: int, dimensions: Tuple[int, ...]) -> Tuple[int, ...]:
    """Rank -> mesh coordinates; dimension 0 is the fastest-varying digit
    (mercury/backend/pytorch/utils.py:41-66)."""
    coords = []
    rest = one_dim_index
    for size in dimensions:
        coords.append(rest % size)
        rest //= size
    return tuple(coords)


@lru_cache(maxsize=None)
def n_dim_to_one_dim(n_dim_index: Tuple[int, ...], dimensions: Tuple[int, ...]) -> int:
    """Inverse of :func:`one_dim_to_n_dim` (mercury/backend/pytorch/utils.py:68-82)."""
    rank, weight = 0, 1
    for idx, size in zip(n_dim_index, dimensions):
        rank += idx * weight
        weight *= size
    return rank


@lru_cache(maxsize=None)
def shift_tuple_element(original_tuple: tuple, index: int, value: int, modulo: int) -> tuple:
    """Coordinates with element ``index`` moved by ``value`` modulo ``modulo``
    (mercury/backend/pytorch/utils.py:84-106)."""
    moved = (original_tuple[index] + value) % modulo
    return original_tuple[:index] + (moved,) + original_tuple[index + 1:]


def get_src_dst_ranks(indices: Tuple[int, ...], mesh_shape: Tuple[int, ...],
                      ring_dims: Sequence[int]) -> Tuple[int, int]:
    """Final write-back hop of a ringed reduce buffer (mercury/backend/pytorch/utils.py:171-192):
    walking ``ring_dims`` from the last to the first, shift by 1 on the last and by the previous
    dimension's size on each earlier one; the source is that shift backwards, the destination
    forwards."""
    src, dst = tuple(indices), tuple(indices)
    step = 1
    for dim in reversed(list(ring_dims)):
        src = shift_tuple_element(src, dim, -step, mesh_shape[dim])
        dst = shift_tuple_element(dst, dim, step, mesh_shape[dim])
        step = mesh_shape[dim]
    return n_dim_to_one_dim(src, tuple(mesh_shape)), n_dim_to_one_dim(dst, tuple(mesh_shape))


def reduce_buffer_route(mesh_shape: Sequence[int]) -> Tuple[List[List[int]], List[int]]:
    """Route of a ringed reduce buffer over the mesh (codegen.py:116-190): ``sends[s][r]`` is the rank
    that rank ``r`` sends its buffer to after step ``s`` (innermost mesh dimension first, a hop on the
    next dimension when the inner ring wraps), ``home[r]`` the destination of the write-back hop that
    rank ``r`` makes after the last step (``get_src_dst_ranks``)."""
    mesh_shape = tuple(int(x) for x in mesh_shape)
    world = 1
    for m in mesh_shape:
        world *= m
    sends: List[List[int]] = []
    idx = [0] * len(mesh_shape)
    for _ in range(world - 1):
        dim = next(d for d in range(len(mesh_shape)) if idx[d] + 1 != mesh_shape[d])
        sends.append([n_dim_to_one_dim(shift_tuple_element(one_dim_to_n_dim(r, mesh_shape), dim, 1, mesh_shape[dim]),
                                       mesh_shape) for r in range(world)])
        for d in range(len(mesh_shape)):      # advance the odometer (dimension 0 fastest)
            idx[d] += 1
            if idx[d] < mesh_shape[d]:
                break
            idx[d] = 0
    dims = list(range(len(mesh_shape)))
    home = [get_src_dst_ranks(one_dim_to_n_dim(r, mesh_shape), mesh_shape, dims)[1] for r in range(world)]
    return sends, home


# ------------------------------------------------------------------------------------------------
# chunk order seen by one rank
# ------------------------------------------------------------------------------------------------
def single_ring_order(rank: int, world: int) -> List[int]:
    """Chunk ids in the order rank ``rank`` computes on them: a hop sends to ``rank + 1`` and
    receives from ``rank - 1`` (codegen.py:480-491), chunk id = the rank it started on."""
    ring = LocalRing((world,), rank)
    order = [ring.current]
    for _ in range(world - 1):
        ring.hop(0)
        order.append(ring.current)
    return order


def double_ring_order(rank: int, inner: int, outer: int) -> List[int]:
    """Order on an ``(inner, outer)`` mesh: ``for outer: for inner:`` with a hop along mesh
    dimension 0 unless the inner loop is at its last step, then one along dimension 1
    (codegen.py:480-491 for two RingComms on one tensor dimension, tests/test_double_ring.py:56-84)."""
    ring = LocalRing((inner, outer), rank)
    order = []
    for o in range(outer):
        for i in range(inner):
            order.append(ring.current)
            if i + 1 != inner:
                ring.hop(0)
            elif o + 1 != outer:
                ring.hop(1)
    return order


def ring_divide_order(rank: int, world: int, divide: int) -> List[Tuple[int, int]]:
    """(chunk, sub-chunk) pairs for ``ring_divide = divide``: the sub-chunk loop wraps the ring loop
    (codegen.py:299-306), so each sub-chunk makes a full trip round the ring before the next."""
    return [(c, s) for s in range(divide) for c in single_ring_order(rank, world)]


def zigzag_blocks(rank: int, world: int) -> Tuple[int, int]:
    """Causal load balancing: rank r holds sequence blocks r and 2W-1-r of 2W equal blocks."""
    return rank, 2 * world - 1 - rank


def zigzag_step(rank: int, step: int, world: int) -> Tuple[str, int]:
    """Mask class of ring step ``step``: the chunk that started on ``src`` holds blocks ``src`` and
    ``2W-1-src``.  Step 0 is the local square (causal); an earlier rank's chunk (src < rank) is
    fully visible in its first block and hidden in its second; a later rank's chunk is hidden from
    the rank's first Q block and fully visible to its second."""
    src = single_ring_order(rank, world)[step]
    if step == 0:
        return "diag", src
    return ("kv_first_half", src) if src < rank else ("q_second_half", src)


class LocalRing:
    """Single-process replay of the neighbour exchange (stand-in for ``SendRecv``,
    mercury/backend/pytorch/utils.py:9-39).

    It tracks which rank's original chunk every rank of the mesh currently holds.  ``hop(dim)``
    moves all of them one step along mesh dimension ``dim`` (everyone sends to ``+1`` and receives
    from ``-1``).  With ``chunks`` given, ``send_recv/commit/wait`` mirror the reference protocol --
    including its misuse errors -- and ``send_recv`` returns the tensor the emulated rank would
    have received.
    """

    def __init__(self, mesh_shape: Sequence[int], rank: int,
                 chunks: Optional[Sequence[torch.Tensor]] = None, copy: bool = False):
        self.mesh_shape = tuple(int(x) for x in mesh_shape)
        self.world = 1
        for s in self.mesh_shape:
            self.world *= s
        if not 0 <= rank < self.world:
            raise ValueError(f"rank {rank} outside a mesh of {self.world} ranks")
        if chunks is not None and len(chunks) != self.world:
            raise ValueError("need one chunk per rank")
        self.rank = rank
        self.chunks = chunks
        self.copy = copy
        self.held = list(range(self.world))       # held[r] = id of the chunk rank r has now
        self._pending = False
        self._committed = False

    @property
    def current(self) -> int:
        return self.held[self.rank]

    def current_chunk(self) -> torch.Tensor:
        return self.chunks[self.current]

    def hop(self, dim: int) -> int:
        size = self.mesh_shape[dim]
        nxt = list(self.held)
        for r in range(self.world):
            to = n_dim_to_one_dim(shift_tuple_element(one_dim_to_n_dim(r, self.mesh_shape), dim, 1, size),
                                  self.mesh_shape)
            nxt[to] = self.held[r]
        self.held = nxt
        return self.current

    # -- SendRecv protocol -------------------------------------------------------------------------
    def send_recv(self, to_rank: int, from_rank: int, send_tensor: torch.Tensor,
                  recv_tensor: Optional[torch.Tensor] = None) -> torch.Tensor:
        mine = one_dim_to_n_dim(self.rank, self.mesh_shape)
        to = one_dim_to_n_dim(to_rank, self.mesh_shape)
        moved = [d for d in range(len(mine)) if mine[d] != to[d]]
        if len(moved) > 1:
            raise RuntimeError("a ring hop moves along exactly one mesh dimension")
        if moved:
            dim = moved[0]
            if shift_tuple_element(mine, dim, 1, self.mesh_shape[dim]) != to or \
               shift_tuple_element(mine, dim, -1, self.mesh_shape[dim]) != one_dim_to_n_dim(from_rank, self.mesh_shape):
                raise RuntimeError("LocalRing only replays hops that send to +1 and receive from -1")
            self.hop(dim)
        self._pending = True
        got = self.chunks[self.current] if self.chunks is not None else send_tensor
        if recv_tensor is not None:
            recv_tensor.copy_(got)
            return recv_tensor
        return got.clone() if self.copy else got

    def commit(self) -> None:
        if self._committed:
            raise RuntimeError("commit called twice")
        self._committed = True

    def wait(self) -> None:
        if not self._committed:
            raise RuntimeError("wait called before commit")
        self._committed = False
        self._pending = False
