"""Rank <-> mesh index arithmetic and the local stand-in for the ring exchange.

The generated ring code gets these by ``from mercury.backend import *``
(mercury/backend/pytorch/utils.py:9-106,171-192).  On one GPU there is no peer to exchange with:
``LocalRing`` holds every rank's KV chunk, replays the hops all ranks would make together, and
hands the emulated rank the chunk it would have received -- buffer rotation in place of send/recv.
"""
from __future__ import annotations

import contextlib
import queue
import threading
from functools import lru_cache
from typing import Callable, List, Optional, Sequence, Tuple

import torch

__all__ = ["one_dim_to_n_dim", "n_dim_to_one_dim", "shift_tuple_element", "get_src_dst_ranks",
           "get_device_group", "debug_print", "LocalGroup", "local_peers", "LocalMesh", "LocalRing", "single_ring_order", "double_ring_order", "ring_divide_order",
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


# ------------------------------------------------------------------------------------------------
# communication groups of a collective, and their single-GPU stand-in
# ------------------------------------------------------------------------------------------------
_PEER_SOURCE: List[Optional[Callable[[int], torch.Tensor]]] = [None]
_ACTIVE_MESH: List[Optional["LocalMesh"]] = [None]


@contextlib.contextmanager
def local_peers(source: Callable[[int], torch.Tensor]):
    """While the block runs, the groups ``get_device_group`` hands out take the operands of the ranks that are not
    the calling one from ``source(rank)``: on one GPU there is no peer to reduce with, so whoever emulates a
    mesh says what the other ranks would contribute (their partial results as they are when the collective
    starts)."""
    before = _PEER_SOURCE[0]
    _PEER_SOURCE[0] = source
    try:
        yield
    finally:
        _PEER_SOURCE[0] = before


class LocalGroup:
    """Single-GPU stand-in for the process group of a collective.  Either ``peers`` -- the operands of all ranks
    of the group as they are when the collective starts, ``rank`` the position of the calling rank among them --
    or, as ``get_device_group`` builds it, the global ``ranks`` of the group: the operands of the other ranks
    are then asked of the source installed by ``local_peers`` when the collective runs."""

    def __init__(self, peers: Optional[Sequence[torch.Tensor]] = None, rank: int = 0,
                 ranks: Optional[Sequence[int]] = None):
        if peers is None and ranks is None:
            raise ValueError("a group needs the operands of its ranks or their rank numbers")
        n = len(peers) if peers is not None else len(ranks)
        if not 0 <= rank < n:
            raise ValueError("rank outside the group")
        self.peers = list(peers) if peers is not None else None
        self.ranks = tuple(ranks) if ranks is not None else tuple(range(n))
        self.rank = rank

    def size(self) -> int:
        return len(self.ranks)

    def operands(self, mine: torch.Tensor) -> List[torch.Tensor]:
        """Operands of all ranks of the group, the calling rank's being ``mine``."""
        if self.peers is not None:
            return list(self.peers)
        if _ACTIVE_MESH[0] is not None:
            return _ACTIVE_MESH[0]._gather(self.ranks, mine)
        source = _PEER_SOURCE[0]
        if source is None and len(self.ranks) > 1:
            raise RuntimeError("this group was built by get_device_group on one GPU: run the collective inside "
                               "`with local_peers(source):` so that the other ranks' operands are known")
        return [mine if i == self.rank else source(r) for i, r in enumerate(self.ranks)]


@lru_cache(maxsize=None)
def get_device_group(indices: Tuple[int, ...], mesh_shape: Tuple[int, ...], dims: Tuple[int, ...], debug: bool = False):
    """Communication group of the rank at mesh coordinates ``indices`` over the mesh dimensions ``dims``
    (mercury/backend/pytorch/utils.py:114-169): all ranks whose coordinates agree with ``indices`` outside
    ``dims``.  ``debug=True`` returns their sorted rank numbers, as the reference does; otherwise the reference
    returns a ``dist.new_group`` of them, and this build, which runs one rank per process on one GPU, a
    ``LocalGroup`` over the same ranks (see ``local_peers``)."""
    indices, mesh_shape, dims = tuple(indices), tuple(mesh_shape), tuple(dims)
    for dim in dims:
        if dim < 0 or dim >= len(mesh_shape):
            raise ValueError(f"Invalid dimension index: {dim}, mesh shape: {mesh_shape}")
    members = [indices]
    for dim in dims:
        members = [m[:dim] + (i,) + m[dim + 1:] for m in members for i in range(mesh_shape[dim])]
    ranks = tuple(sorted({n_dim_to_one_dim(m, mesh_shape) for m in members}))
    if debug:
        return ranks
    return LocalGroup(ranks=ranks, rank=ranks.index(n_dim_to_one_dim(indices, mesh_shape)))


def debug_print(*args) -> None:
    """``print`` with the rank in front, one rank after the other (mercury/backend/pytorch/utils.py:108-112);
    without an initialised process group there is one rank and nothing to take turns with."""
    import torch.distributed as dist

    if not (dist.is_available() and dist.is_initialized()):
        print("[Rank 0]", *args)
        return
    for rank in range(dist.get_world_size()):
        if rank == dist.get_rank():
            print(f"[Rank {rank}]", *args)
        dist.barrier()


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


class LocalMesh:
    """Every rank of a mesh as one thread of this process, all on the one GPU and on one stream: what a multi-rank
    launch of a generated step function does, replayed where there is a single device.  ``run(fn)`` calls
    ``fn(rank)`` in one thread per rank; inside, ``dist`` stands in for ``torch.distributed`` (``get_rank`` is the
    thread's rank), ``SendRecv()`` gives an object with the reference's ``send_recv / commit / wait`` protocol
    (mercury/backend/pytorch/utils.py:9-39) whose messages travel through per-pair mailboxes, and the groups of
    ``get_device_group`` gather the operands of their ranks when a collective runs.  A message is a copy taken at
    ``commit`` (as on a wire); since all threads enqueue on one stream, a receiver's copy is ordered behind the
    kernels that produced the message.  Nothing blocks for longer than ``timeout`` seconds: a rank that waits for
    a message nobody sends raises instead of hanging."""

    def __init__(self, mesh_shape: Sequence[int], timeout: float = 60.0):
        self.mesh_shape = tuple(int(x) for x in mesh_shape)
        self.world = 1
        for m in self.mesh_shape:
            self.world *= m
        self.timeout = timeout
        self._tls = threading.local()
        self._mail = {}
        self._lock = threading.Lock()
        self._gathers = {}
        self._world_barrier = threading.Barrier(self.world)
        self._failed = threading.Event()          # set by the first rank that raises: the others stop waiting
        mesh = self

        class _Dist:
            """The few names of torch.distributed that generated code touches."""

            @staticmethod
            def get_rank() -> int:
                return mesh.rank()

            @staticmethod
            def get_world_size() -> int:
                return mesh.world

            @staticmethod
            def barrier() -> None:
                mesh._world_barrier.wait(mesh.timeout)

            @staticmethod
            def all_reduce(*args, **kwargs):
                raise RuntimeError("collectives run inside update_out_and_lse_collective / add_collective")

            @staticmethod
            def reduce(*args, **kwargs):
                raise RuntimeError("collectives run inside update_out_and_lse_collective / add_collective")

        self.dist = _Dist

    def rank(self) -> int:
        return self._tls.rank

    def _box(self, src: int, dst: int) -> "queue.Queue":
        with self._lock:
            return self._mail.setdefault((src, dst), queue.Queue())

    def SendRecv(self) -> "_MeshSendRecv":
        return _MeshSendRecv(self)

    def _gather(self, ranks: Tuple[int, ...], mine: torch.Tensor) -> List[torch.Tensor]:
        """Operands of all ranks of a group, each a copy taken when its rank arrived at the collective."""
        with self._lock:
            slot = self._gathers.get(ranks)
            if slot is None:
                slot = self._gathers[ranks] = {"barrier": threading.Barrier(len(ranks)), "parts": {}}
        slot["parts"][self.rank()] = mine.clone()
        slot["barrier"].wait(self.timeout)
        parts = [slot["parts"][r] for r in ranks]
        slot["barrier"].wait(self.timeout)          # everyone has read before the next collective writes
        return parts

    def run(self, fn: Callable[[int], object], ranks: Optional[Sequence[int]] = None) -> List[object]:
        """``fn(rank)`` for every rank (or the given ones) at once; returns their results in rank order and
        re-raises the first exception of any rank."""
        ranks = list(range(self.world)) if ranks is None else list(ranks)
        results = {}
        errors = []                                # (rank, exception) in the order they happened
        # a fresh start: nothing of an earlier run (undelivered messages, barriers a failure broke) is left over
        self._failed.clear()
        self._mail, self._gathers = {}, {}
        self._world_barrier = threading.Barrier(self.world)
        device = torch.cuda.current_device() if torch.cuda.is_available() else None
        stream = torch.cuda.current_stream() if torch.cuda.is_available() else None

        def body(r):
            self._tls.rank = r
            try:
                if device is not None:
                    torch.cuda.set_device(device)
                    with torch.cuda.stream(stream):
                        results[r] = fn(r)
                else:
                    results[r] = fn(r)
            except BaseException as exc:          # noqa: BLE001 -- handed to the caller below
                with self._lock:
                    errors.append((r, exc))
                self._failed.set()
                for slot in list(self._gathers.values()):
                    slot["barrier"].abort()
                self._world_barrier.abort()

        if _ACTIVE_MESH[0] is not None:
            raise RuntimeError("a LocalMesh is already running")
        _ACTIVE_MESH[0] = self
        try:
            threads = [threading.Thread(target=body, args=(r,), daemon=True) for r in ranks]
            for t in threads:
                t.start()
            for t in threads:
                t.join()
        finally:
            _ACTIVE_MESH[0] = None
        if errors:
            # the first thing that went wrong, not what the other ranks ran into because of it
            own = [exc for _, exc in errors if not isinstance(exc, (threading.BrokenBarrierError, _PeerFailed))]
            raise own[0] if own else errors[0][1]
        return [results[r] for r in ranks]


class _PeerFailed(RuntimeError):
    """Raised in a rank that was waiting for a message when another rank of the mesh failed."""


class _MeshSendRecv:
    """``SendRecv`` of one rank of a ``LocalMesh``: same calls, same misuse errors as the reference's."""

    def __init__(self, mesh: LocalMesh):
        self._mesh = mesh
        self._ops = []
        self._committed = False

    def send_recv(self, to_rank: int, from_rank: int, send_tensor: torch.Tensor,
                  recv_tensor: Optional[torch.Tensor] = None) -> torch.Tensor:
        res = torch.empty_like(send_tensor) if recv_tensor is None else recv_tensor
        self._ops.append((to_rank, from_rank, send_tensor.contiguous(), res))
        return res

    def commit(self) -> None:
        if self._committed:
            raise RuntimeError("commit called twice")
        me = self._mesh.rank()
        for to_rank, _, send_tensor, _ in self._ops:
            self._mesh._box(me, to_rank).put(send_tensor.clone())
        self._committed = True

    def wait(self) -> None:
        if not self._committed:
            raise RuntimeError("wait called before commit")
        me = self._mesh.rank()
        for _, from_rank, _, res in self._ops:
            box, waited, got = self._mesh._box(from_rank, me), 0.0, None
            while got is None:
                if self._mesh._failed.is_set():
                    raise _PeerFailed(f"rank {me} stopped waiting for rank {from_rank}: another rank raised")
                try:
                    got = box.get(timeout=0.05)
                except queue.Empty:
                    waited += 0.05
                    if waited >= self._mesh.timeout:
                        raise RuntimeError(f"rank {me} waited {self._mesh.timeout} s for a message from rank "
                                           f"{from_rank}") from None
            res.copy_(got)
        self._committed = False
        self._ops = []
