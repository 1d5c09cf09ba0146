"""Fixed-schedule drivers of one rank's ring-attention step on one GPU.

Each driver has the argument list of the function Mercury generates from the template of the same
name (utils/flash_attn_dsl.py:127-180, 182-235, 237-291, 345-408; utils/attn_bwd_dsl.py:37-135) plus a
``ring`` keyword: the :class:`~mercury_artifact_amd.schedule.LocalRing` that stands in for the
neighbour exchange.  The body is the loop the code generator emits for that template
(mercury/backend/pytorch/codegen.py:264-355, 443-523): take the current KV chunk, start the hop for
the next one, run the block kernel through ``_flash_attn_forward(**params)``, fold with
``update_out_and_lse``, and store after the last step.

Two defaults of the forward drivers depart from the literal sequence without changing what is computed:
``deferred_merge=True`` keeps the bf16 block results of all chunks and folds them with ONE
``merge_many`` call after the last chunk (the fold is associative; every block output is read once
instead of the fp32 accumulator travelling through memory once per chunk; results agree with the chain
to fp32 rounding), and ``fused_epilogue=True`` lets the last merge of the chain write ``o`` / ``lse``
itself (bit-identical).  ``deferred_merge=False, fused_epilogue=False`` is the generated code's literal
sequence: ``update_out_and_lse`` per chunk, then ``o[...] = _out.to(o.dtype)``,
``lse[...] = _lse.squeeze(-1).transpose(1, 2)``.
"""
from __future__ import annotations

import warnings
from typing import Optional

import torch

from . import _native as N
from .flash_attn_interface import _flash_attn_backward, _flash_attn_forward, attn_bwd_block
from .merge import (MAX_MERGE_MANY, get_default_args, grad_accumulate, merge_into, merge_many, pack_block,
                    unpack_into, update_out_and_lse)
from .schedule import (LocalRing, n_dim_to_one_dim, one_dim_to_n_dim, reduce_buffer_route, shift_tuple_element,
                       zigzag_step)

__all__ = ["flash_attn_pack_kv", "gqa_pack_kv", "flash_attn_pack_split_kv", "flash_attn_expose_reduce",
           "flash_attn_expose_reduce_q_ring",
           "flash_attn_backward", "zigzag_causal_pack_kv", "fp8_pack_split_kv", "quantize_e4m3"]


def _hops(ring: LocalRing):
    """(dim, is_last) per step in generated-loop order: innermost mesh dimension first, a hop on
    the next dimension when the inner loop wraps, nothing after the very last step."""
    shape = ring.mesh_shape
    total = ring.world
    idx = [0] * len(shape)
    for step in range(total):
        hop = None
        for d in range(len(shape)):
            if idx[d] + 1 != shape[d]:
                hop = d
                break
        yield hop
        # advance the odometer (dimension 0 fastest)
        for d in range(len(shape)):
            idx[d] += 1
            if idx[d] < shape[d]:
                break
            idx[d] = 0


def _neighbours(ring: LocalRing, dim: int):
    me = one_dim_to_n_dim(ring.rank, ring.mesh_shape)
    size = ring.mesh_shape[dim]
    send_to = n_dim_to_one_dim(shift_tuple_element(me, dim, 1, size), ring.mesh_shape)
    recv_from = n_dim_to_one_dim(shift_tuple_element(me, dim, -1, size), ring.mesh_shape)
    return send_to, recv_from


def _fwd_params(q, k, v, softmax_scale, dropout_p, causal, window_size, alibi_slopes, **extra):
    params = get_default_args(_flash_attn_forward).copy()
    params.update({
        "q": q, "k": k, "v": v,
        "dropout_p": dropout_p,
        "softmax_scale": softmax_scale,
        "causal": causal,
        "alibi_slopes": alibi_slopes,
        "return_softmax": True and dropout_p > 0,
        "window_size_left": window_size[0],
        "window_size_right": window_size[1],
    })
    params.update(extra)
    return params


_SIDE_STREAMS = {}


def _side_stream(device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority), made on first use and kept."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return _SIDE_STREAMS[key]


def _ring_forward(q, kv, o, lse, softmax_scale, dropout_p, causal, window_size, alibi_slopes,
                  ring: LocalRing, fused_epilogue: bool, deferred_merge: bool, ring_divide: int = 1,
                  two_streams: bool = False, **extra):
    """The chunk loop of the forward templates.  ``ring_divide = k > 1`` is the schedule option of the same
    name (mercury/backend/pytorch/codegen.py:299-306): an outer loop over k sub-chunks of the KV rows wraps
    the ring loop, so the step makes k * W block calls on (Sq x Sc / k) blocks and every hop moves 1/k of a
    chunk.

    ``two_streams`` (with the deferred fold only, where the block launches do not depend on each other): every
    other block launch goes to a second stream, so that the tail of one launch (workgroups of its last round,
    drained pipelines) overlaps the head of the next; the fold waits for both.  The side stream starts behind
    everything queued on the current stream when the step begins, and a block launched there waits for the event
    recorded on the current stream right behind the hop that delivers its chunk (so for the hop's copy, not for the
    block launch that follows it on the current stream)."""
    blocks = []
    _out = None
    _lse = None
    _kv = None
    _next_kv = None
    steps = list(_hops(ring))
    ring_divide = int(ring_divide)
    Sc = kv.shape[2]
    if ring_divide < 1 or Sc % ring_divide:
        raise ValueError("ring_divide must divide the chunk's rows")
    if ring_divide > 1 and ring.chunks is None:
        raise ValueError("ring_divide needs a LocalRing that holds the chunks")
    sub = Sc // ring_divide
    n_blocks = len(steps) * ring_divide
    defer = (deferred_merge and n_blocks <= MAX_MERGE_MANY and o.dtype == torch.bfloat16
             and o.is_contiguous() and lse.is_contiguous())
    if deferred_merge and not defer:
        warnings.warn(f"ring step of {n_blocks} blocks into a {o.dtype} output: the one-pass fold takes at most "
                      f"{MAX_MERGE_MANY} blocks and writes contiguous bfloat16, so this step merges block by block "
                      "(same result, one pass over the fp32 accumulator per block)", RuntimeWarning, stacklevel=3)
    done = 0
    main = side = None
    kv_ready = next_ready = None
    if two_streams and defer:
        main = torch.cuda.current_stream(q.device)
        side = _side_stream(q.device)
        side.wait_stream(main)
    for part in range(ring_divide):
        rows = slice(part * sub, (part + 1) * sub)
        part_ring = ring if ring_divide == 1 else \
            LocalRing(ring.mesh_shape, ring.rank, [c[:, :, rows] for c in ring.chunks], copy=ring.copy)
        for step, hop in enumerate(steps):
            if step == 0:
                _kv = kv[:, :, rows].contiguous()
                kv_ready = None
                if side is not None and part > 0:      # the sub-chunk copy above sits behind earlier launches
                    kv_ready = torch.cuda.Event()
                    kv_ready.record(main)
            else:
                part_ring.wait()
                _kv = _next_kv
                kv_ready = next_ready
            if hop is not None:
                send_to, recv_from = _neighbours(part_ring, hop)
                _next_kv = part_ring.send_recv(send_to, recv_from, _kv)
                part_ring.commit()
                next_ready = None
                if side is not None:                   # what the hop enqueued on the current stream ends here
                    next_ready = torch.cuda.Event()
                    next_ready.record(main)
            _k = _kv[0]
            _v = _kv[1]
            params = _fwd_params(q, _k, _v, softmax_scale, dropout_p, causal, window_size, alibi_slopes, **extra)
            if side is not None and done % 2 == 1:
                if kv_ready is not None:
                    side.wait_event(kv_ready)
                _kv.record_stream(side)              # may have been allocated by the hop on the current stream
                with torch.cuda.stream(side):
                    outputs = _flash_attn_forward(**params)
                for t in outputs[:2]:
                    t.record_stream(main)            # allocated under the side stream, read by the fold on the main one
            else:
                outputs = _flash_attn_forward(**params)
            assert len(outputs) == 4
            block_out, block_lse, _, _ = outputs
            done += 1
            if defer:
                blocks.append((block_out, block_lse))
                if done == n_blocks:
                    if side is not None:
                        main.wait_stream(side)
                    merge_many([b[0] for b in blocks], [b[1] for b in blocks], o, lse)
                    return
                continue
            if fused_epilogue and done == n_blocks:
                # last merge writes o / lse directly (same arithmetic, two passes fewer)
                merge_into(_out, _lse, block_out, block_lse, None, None, o, lse)
                return
            _out, _lse = update_out_and_lse(_out, _lse, block_out, block_lse)
    o[:, :, :, :] = _out.to(o.dtype)
    lse[:, :, :] = _lse.squeeze(dim=-1).transpose(1, 2)


def flash_attn_pack_kv(q, kv, o, lse, softmax_scale, dropout_p=0, causal=False, window_size=(-1, -1),
                       alibi_slopes=None, deterministic=False, *, ring: LocalRing,
                       fused_epilogue: bool = True, deferred_merge: bool = True, ring_divide: int = 1,
                       two_streams: bool = False):
    """Single-ring forward step (template utils/flash_attn_dsl.py:127-180).  q (B,Sq,H,D), kv the
    rank's own (2,B,Sc,H,D), o (B,Sq,H,D) and lse (B,H,Sq) are written."""
    _ring_forward(q, kv, o, lse, softmax_scale, dropout_p, causal, window_size, alibi_slopes, ring,
                  fused_epilogue, deferred_merge, ring_divide, two_streams)


def gqa_pack_kv(q, kv, o, lse, softmax_scale, dropout_p=0, causal=False, window_size=(-1, -1),
                alibi_slopes=None, deterministic=False, *, ring: LocalRing, fused_epilogue: bool = True,
                deferred_merge: bool = True, ring_divide: int = 1):
    """GQA forward step (template utils/flash_attn_dsl.py:182-235): kv has Hkv heads, q has
    Hkv * HEADS_PER_GROUP; the block kernel maps q head h to kv head h // HEADS_PER_GROUP."""
    _ring_forward(q, kv, o, lse, softmax_scale, dropout_p, causal, window_size, alibi_slopes, ring,
                  fused_epilogue, deferred_merge, ring_divide)


def flash_attn_pack_split_kv(q, kv, o, lse, softmax_scale, dropout_p=0, causal=False,
                             window_size=(-1, -1), alibi_slopes=None, deterministic=False, *,
                             ring: LocalRing, fused_epilogue: bool = True, deferred_merge: bool = True,
                             ring_divide: int = 1):
    """Double-ring forward step (template utils/flash_attn_dsl.py:237-291): ``ring`` is built on the
    2-D mesh ``(inner, outer)``; the loop order and hops follow from the mesh shape."""
    if len(ring.mesh_shape) != 2:
        raise ValueError("the double ring needs a 2-D mesh (inner, outer)")
    _ring_forward(q, kv, o, lse, softmax_scale, dropout_p, causal, window_size, alibi_slopes, ring,
                  fused_epilogue, deferred_merge, ring_divide)


def _store_packed(buf, o, lse, fused: bool):
    """The stores after the managed reduction (utils/flash_attn_dsl.py:406-407): one kernel, or the literal
    torch expressions."""
    if fused and o.dtype == torch.bfloat16 and o.is_contiguous() and lse.is_contiguous() and o.shape[-1] % 8 == 0 \
            and 256 % (o.shape[-1] // 8) == 0:
        unpack_into(buf, o, lse)
        return
    o[:, :, :, :] = buf[..., :-1].to(o.dtype)
    lse[:, :, :] = buf[..., -1].transpose(1, 2)


def flash_attn_expose_reduce(q, kv, o, lse, softmax_scale, dropout_p=0, causal=False,
                             window_size=(-1, -1), alibi_slopes=None, deterministic=False, *,
                             ring: LocalRing, fused_epilogue: bool = True):
    """Managed-reduction form (template utils/flash_attn_dsl.py:345-408) with the KV ring: block
    results are packed ``(out | lse)`` and folded by ``flash_reduce``; pack and reduce run as one
    kernel."""
    buf = None
    _kv = None
    _next_kv = None
    for step, hop in enumerate(_hops(ring)):
        if step == 0:
            _kv = kv.contiguous()
        else:
            ring.wait()
            _kv = _next_kv
        if hop is not None:
            send_to, recv_from = _neighbours(ring, hop)
            _next_kv = ring.send_recv(send_to, recv_from, _kv)
            ring.commit()
        outputs = _flash_attn_forward(**_fwd_params(q, _kv[0], _kv[1], softmax_scale, dropout_p, causal,
                                                    window_size, alibi_slopes))
        assert len(outputs) == 4
        block_out, block_lse, _, _ = outputs
        buf = pack_block(block_out, block_lse, reduce_into=buf)
    _store_packed(buf, o, lse, fused_epilogue)


def flash_attn_expose_reduce_q_ring(qs, kvs, os_, lses, softmax_scale, dropout_p=0, causal=False,
                                    window_size=(-1, -1), alibi_slopes=None, deterministic=False, *,
                                    mesh_shape=None, fused_epilogue: bool = True):
    """The managed-reduction template (utils/flash_attn_dsl.py:345-408) scheduled as a ring over the
    *reduce buffer*: every rank keeps its KV shard, Q and the packed partial result ``(out | lse)``
    travel (codegen.py:116-190).  A rank's step is: block forward of the Q that just arrived against
    the local KV, ``buf = flash_reduce(arrived_partial, pack(block))`` (one fused kernel), send on;
    after the last step the buffer makes the write-back hop of ``get_src_dst_ranks``
    (mercury/backend/pytorch/utils.py:171-192) to the rank that owns its Q rows.

    What arrives at a rank was computed by the other ranks, so this driver runs ALL ranks of the mesh
    in lock step on the one GPU: ``qs[r]``, ``kvs[r]`` are rank r's shards, ``os_[r]`` / ``lses[r]``
    receive its result.  One rank's share of the work is 1 / world of the launches."""
    world = len(qs)
    mesh_shape = tuple(mesh_shape) if mesh_shape is not None else (world,)
    sends, home_of = reduce_buffer_route(mesh_shape)
    if len(home_of) != world or not (len(kvs) == len(os_) == len(lses) == world):
        raise ValueError("need one q, kv, o and lse per rank of the mesh")
    q_cur = list(qs)
    arrived = [None] * world
    home = [None] * world
    for step in range(world):
        buf = []
        for r in range(world):
            kv = kvs[r]
            outputs = _flash_attn_forward(**_fwd_params(q_cur[r], kv[0], kv[1], softmax_scale, dropout_p, causal,
                                                        window_size, alibi_slopes))
            assert len(outputs) == 4
            block_out, block_lse, _, _ = outputs
            buf.append(pack_block(block_out, block_lse, reduce_into=arrived[r]))
        if step + 1 != world:
            q_next, arrived = [None] * world, [None] * world
            for r in range(world):
                q_next[sends[step][r]], arrived[sends[step][r]] = q_cur[r], buf[r]
            q_cur = q_next
        else:
            for r in range(world):
                home[home_of[r]] = buf[r]
    for r in range(world):
        _store_packed(home[r], os_[r], lses[r], fused_epilogue)


def zigzag_causal_pack_kv(q, kv, o, lse, softmax_scale, dropout_p=0, causal=True, window_size=(-1, -1),
                          alibi_slopes=None, deterministic=False, *, ring: LocalRing, deferred_merge: bool = True):
    """Causal forward step in the zigzag layout (rank r holds sequence blocks r and 2W-1-r).  Not in
    the reference, which only carries the ``slice_`` hook (utils/flash_attn_dsl.py:56,63-68); the
    three step classes are the diagonal (causal block), "first half of the chunk" and "second half
    of the Q rows" (merged through ``slice_``)."""
    if len(ring.mesh_shape) != 1:
        raise ValueError("zigzag runs on a 1-D ring")
    world = ring.world
    Sq = q.shape[1]
    if Sq % 2 or kv.shape[2] != Sq:
        raise ValueError("zigzag needs an even number of local rows and equal Q / KV shards")
    half = Sq // 2
    _out = _lse = _kv = _next_kv = None
    defer = (deferred_merge and world <= MAX_MERGE_MANY and o.dtype == torch.bfloat16
             and o.is_contiguous() and lse.is_contiguous())
    blocks = []
    for step in range(world):
        if step == 0:
            _kv = kv.contiguous()
        else:
            ring.wait()
            _kv = _next_kv
        if step + 1 != world:
            send_to, recv_from = _neighbours(ring, 0)
            _next_kv = ring.send_recv(send_to, recv_from, _kv)
            ring.commit()
        kind, _ = zigzag_step(ring.rank, step, world)
        if kind == "diag":
            bq, bk, bv, bc, sl = q, _kv[0], _kv[1], True, None
        elif kind == "kv_first_half":
            bq, bk, bv, bc, sl = q, _kv[0][:, :half], _kv[1][:, :half], False, None
        else:
            bq, bk, bv, bc, sl = q[:, half:], _kv[0], _kv[1], False, (slice(None), slice(half, None))
        outputs = _flash_attn_forward(**_fwd_params(bq, bk, bv, softmax_scale, dropout_p, bc,
                                                    window_size, alibi_slopes))
        block_out, block_lse, _, _ = outputs
        if defer:
            blocks.append((block_out, block_lse, 0 if sl is None else half))
            continue
        _out, _lse = update_out_and_lse(_out, _lse, block_out, block_lse, slice_=sl)
    if defer:
        merge_many([b[0] for b in blocks], [b[1] for b in blocks], o, lse, row_begin=[b[2] for b in blocks])
        return
    o[:, :, :, :] = _out.to(o.dtype)
    lse[:, :, :] = _lse.squeeze(dim=-1).transpose(1, 2)


def quantize_e4m3(x: torch.Tensor):
    """Per-tensor e4m3 quantisation through mhip_quantize_e4m3: scale s = amax / 448 (fp32; 1 for an all-zero
    tensor), x_q = round-to-nearest-even(clamp(x / s, -448, 448)) as ``torch.float8_e4m3fn``.  Returns
    ``(x_q, s)`` with ``s`` a 0-dim fp32 tensor on the device (the block kernel's descale).  fp32 or bf16
    input on the GPU."""
    N.require_cuda(x)
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise RuntimeError("quantize_e4m3 takes float32 or bfloat16")
    xc = x.contiguous()
    xq = torch.empty(xc.shape, dtype=torch.float8_e4m3fn, device=x.device)
    ws = torch.empty(2, dtype=torch.float32, device=x.device)          # [scale, scratch for the maximum]
    with torch.cuda.device(x.device):
        code = N.lib().mhip_quantize_e4m3(N.ptr(xc), N.MHIP_F32 if x.dtype == torch.float32 else N.MHIP_BF16,
                                          xc.numel(), N.ptr(xq), ws.data_ptr(), ws.data_ptr() + 4, N.stream_of(xc))
    N.check(code, "mhip_quantize_e4m3")
    return xq, ws[0]


def fp8_pack_split_kv(q, kv, o, lse, softmax_scale, q_descale, k_descale, v_descale, dropout_p=0,
                      causal=False, window_size=(-1, -1), alibi_slopes=None, deterministic=False, *,
                      ring: LocalRing, fused_epilogue: bool = True, deferred_merge: bool = True,
                      ring_divide: int = 1):
    """Forward step on e4m3 Q/K/V with per-tensor descales (not in the reference); any mesh."""
    _ring_forward(q, kv, o, lse, softmax_scale, dropout_p, causal, window_size, alibi_slopes, ring,
                  fused_epilogue, deferred_merge, ring_divide, q_descale=q_descale, k_descale=k_descale,
                  v_descale=v_descale)


def flash_attn_backward(q, kv, o, lse, dout, dq, dkv, softmax_scale, dropout_p=0, causal=False,
                        window_size=(-1, -1), alibi_slopes=None, deterministic=False, *,
                        ring: LocalRing, dkv_chunks: Optional[dict] = None, fused_accumulate: bool = True):
    """Backward ring step (template utils/attn_bwd_dsl.py:37-135 after ``shift`` on the KV axis):
    KV chunks arrive in ring order, each gets a block backward against the local q / o / lse / dout;
    dq accumulates in fp32 over the chunks (utils/attn_bwd_dsl.py:117-122) and is stored as
    ``dq.dtype`` at the end (131-132).  The fp32 dK/dV accumulator that travels with its chunk on a
    real ring has exactly one contribution per rank, so here each chunk's block gradient is kept in
    ``dkv_chunks[chunk id]`` (fp32) and the rank's own chunk is stored to ``dkv``.

    ``fused_accumulate=True`` (default) lets the block kernel add its fp32 dq straight into the accumulator
    (one pass fewer over it per chunk, and the sum sees the unrounded block gradient) and casts a chunk's
    dK/dV to fp32 only when ``dkv_chunks`` asks for it; ``False`` is the literal sequence: block backward
    through ``_flash_attn_backward(**params)``, then ``torch.add`` on the bf16 block gradients."""
    if dropout_p != 0 or alibi_slopes is not None or tuple(window_size) != (-1, -1):
        fused_accumulate = False                # let the operator report what it does not support
    reduce_dq = torch.zeros(q.shape, dtype=torch.float32, device=q.device) if fused_accumulate else None
    _kv = _next_kv = None
    own = ring.current
    for step, hop in enumerate(_hops(ring)):
        if step == 0:
            _kv = kv.contiguous()
        else:
            ring.wait()
            _kv = _next_kv
        chunk_id = ring.current
        if hop is not None:
            send_to, recv_from = _neighbours(ring, hop)
            _next_kv = ring.send_recv(send_to, recv_from, _kv)
            ring.commit()
        block_dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        block_dkv = torch.empty(_kv.shape, dtype=kv.dtype, device=kv.device)
        if fused_accumulate:
            attn_bwd_block(dout, q, _kv[0], _kv[1], o, lse, block_dq, block_dkv[0], block_dkv[1], softmax_scale,
                           causal=False, deterministic=deterministic, dq_acc=reduce_dq)
            if dkv_chunks is not None:
                dkv_chunks[chunk_id] = grad_accumulate(None, block_dkv)
            if chunk_id == own:
                dkv[...] = block_dkv
            continue
        params = get_default_args(_flash_attn_backward).copy()
        params.update({
            "dout": dout, "q": q, "k": _kv[0], "v": _kv[1], "out": o, "softmax_lse": lse,
            "dq": block_dq, "dk": block_dkv[0], "dv": block_dkv[1],
            "softmax_scale": softmax_scale, "dropout_p": dropout_p, "causal": False,
            "deterministic": deterministic, "alibi_slopes": alibi_slopes,
        })
        if "window_size" in params:
            params.update({"window_size": window_size})
        else:
            params.update({"window_size_left": window_size[0], "window_size_right": window_size[1]})
        _flash_attn_backward(**params)
        reduce_dq = grad_accumulate(reduce_dq, block_dq)
        red = grad_accumulate(None, block_dkv)
        if dkv_chunks is not None:
            dkv_chunks[chunk_id] = red
        if chunk_id == own:
            dkv[...] = red.to(dkv.dtype)
    dq[...] = reduce_dq.to(dq.dtype)
