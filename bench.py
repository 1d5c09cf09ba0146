#!/usr/bin/env python3
"""Headline benchmark: one rank's bf16 ring-attention forward step on one MI355X.

Workload = the headline bf16 configuration: batch 1, 32 heads, head dim 128, local Q of 4096 rows, 8 KV chunks
of 4096 rows (32768 keys), non-causal, N(0,1) inputs cast to bf16, softmax scale 128^-0.5.
A step = 8 block-forward kernels + ONE fold of the 8 block results into the bf16 output and the (B,H,S) LSE
(the ring drivers' default: the fold is associative, so the chain of 7 LSE merges and the epilogue copies of
the generated code collapse into one pass over the block outputs; that literal chain is timed beside it),
driven through the same block operator Mercury's generated code calls.  Inputs are resident in HBM before
the timed region.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, each counter scaled
# by its reading for the calibration launch at the end of main() (profiles/ring_step_config1_hbm_traffic.md)
TRAFFIC_FWD_BYTES = 134.9e6
TRAFFIC_MERGE_BYTES = 171.5e6
TRAFFIC_MANY_BYTES = 321.0e6


def cpu_baseline(sample_heads: int, B: int, Sq: int, D: int, W: int):
    """The fp32 oracle (a CPU port of the same step) on `sample_heads` of the 32 heads."""
    import torch

    import oracle as O

    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, Sq, sample_heads, D, generator=g)
    kvs = [torch.randn(2, B, Sq, sample_heads, D, generator=g) for _ in range(W)]
    scale = D ** -0.5
    order = O.single_ring_order(0, W)
    O.ring_forward(q[:, :256], [c[:, :, :256] for c in kvs], order, scale)      # warm-up
    t0 = time.perf_counter()
    O.ring_forward(q, kvs, order, scale)
    dt = time.perf_counter() - t0
    flops = 4.0 * B * sample_heads * Sq * Sq * D * W
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{sample_heads} of 32 heads of the same step (Q 4096 x 8 chunks of 4096, fp32 torch "
                      f"matmul/logsumexp + merge), {dt:.1f} s"}


# One rank's forward step as Mercury's generator spells it (mercury/backend/pytorch/codegen.py:264-355, 442-523
# for the template utils/flash_attn_dsl.py:127-180): every name but torch is resolved in the exec namespace.
GENERATED_STEP_TEXT = '''
def generated_ring_step(q, kv, o, lse, softmax_scale, dropout_p=0, causal=False, window_size=(-1, -1),
                        alibi_slopes=None, deterministic=False):
    indices = one_dim_to_n_dim(RANK, (WORLD,))
    _out = None
    _lse = None
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
        assert len(outputs) == 4
        block_out, block_lse, _, _ = outputs
        _out, _lse = update_out_and_lse(_out, _lse, block_out, block_lse)
    o[:, :, :, :] = _out.to(q.dtype)
    lse[:, :, :] = _lse.squeeze(dim=-1).transpose(1, 2)
'''


def operand_dependence(torch, M, dev, shape, scale):
    """The headline block kernel (one chunk, 4096 x 4096) on operands that toggle few bits: all zeros, and small
    integers.  Same kernel, same instruction stream, same number of MFMAs; only the switching activity of the
    data differs, and with it the clock the power management allows."""
    B, Sq, H, D = shape
    out = {}
    flops = 4.0 * B * H * Sq * Sq * D
    for name, make in (("zeros", lambda *s: torch.zeros(*s, device=dev)),
                       ("small_integers", lambda *s: torch.randint(-2, 3, s, device=dev).float())):
        q = make(B, Sq, H, D).bfloat16()
        kv = make(2, B, Sq, H, D).bfloat16()
        o = torch.empty_like(q)
        lse = torch.empty(B, H, Sq, dtype=torch.float32, device=dev)
        for _ in range(5):
            M.attn_fwd_block(q, kv[0], kv[1], scale, out=o, lse=lse)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            M.attn_fwd_block(q, kv[0], kv[1], scale, out=o, lse=lse)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 20
        out[name] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1),
                     "pct_of_bf16_mfma_peak": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS * 100, 2)}
    return out


def smi_snapshot():
    """Socket power and clocks as `amd-smi metric --power --clock` prints them, read while the GPU is busy (the
    caller has work queued).  Best effort: None when the tool is missing or refuses."""
    import re
    import subprocess
    try:
        res = subprocess.run(["amd-smi", "metric", "--power", "--clock"], stdout=subprocess.PIPE,
                             stderr=subprocess.DEVNULL, text=True, timeout=20)
    except (OSError, subprocess.SubprocessError):
        return None
    power = re.search(r"SOCKET_POWER:\s*([0-9.]+)\s*W", res.stdout)
    clocks = [int(x) for x in re.findall(r"^\s*CLK:\s*([0-9]+)\s*MHz", res.stdout, flags=re.M)]
    if not power and not clocks:
        return None
    return {"socket_power_w": float(power.group(1)) if power else None, "clk_mhz_first_entries": clocks[:9]}


def other_kernels(torch, M, dev):
    """Block kernels of the other configurations at their per-rank shapes, HIP events over 10 launches each
    (reported next to the headline, not part of it)."""
    def timeit(fn, n=10, w=3):
        for _ in range(w):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    out = {}
    B, S, H, D = 1, 4096, 32, 128
    scale = D ** -0.5
    q = torch.randn(B, S, H, D, device=dev).bfloat16()
    kv = torch.randn(2, B, S, H, D, device=dev).bfloat16()
    do = torch.randn(B, S, H, D, device=dev).bfloat16()
    o = torch.empty_like(q)
    lse = torch.empty(B, H, S, dtype=torch.float32, device=dev)
    unit = 2.0 * B * H * S * S * D            # one S x S x D product per head
    ms = timeit(lambda: M.attn_fwd_block(q, kv[0], kv[1], scale, causal=True, out=o, lse=lse))
    out["fwd_bf16_causal_4096x4096"] = {"ms": round(ms, 4), "tflops": round(unit / ms / 1e9, 1),
                                        "flops": "4 B H Sq Sc D / 2"}
    M.attn_fwd_block(q, kv[0], kv[1], scale, out=o, lse=lse)
    dq, dkv = torch.empty_like(q), torch.empty_like(kv)
    ms = timeit(lambda: M.attn_bwd_block(do, q, kv[0], kv[1], o, lse, dq, dkv[0], dkv[1], scale))
    out["bwd_bf16_4096x4096"] = {"ms": round(ms, 4), "tflops": round(5 * unit / ms / 1e9, 1),
                                 "pct_of_bf16_mfma_peak": round(5 * unit / ms / 1e9 / 25.0, 2),
                                 "tflops_executed": round(7 * unit / ms / 1e9, 1),
                                 "flops": "10 B H Sq Sc D algorithmic; the two-pass kernel executes 14"}
    # one rank's backward step over the same 8 chunks (dq accumulated in fp32 over the chunks, dk/dv per chunk)
    chunks_b = [kv for _ in range(8)]                       # timing only: every chunk has the same bytes
    ms = timeit(lambda: M.flash_attn_backward(q, kv, o, lse, do, dq, dkv, scale, ring=M.LocalRing((8,), 0, chunks_b)),
                n=3, w=1)
    out["step_bf16_backward_ring_4096x8"] = {"ms": round(ms, 3), "tflops": round(8 * 5 * unit / ms / 1e9, 1),
                                             "flops": "8 chunks x 10 B H Sq Sc D algorithmic"}
    del dq, dkv, do
    S8 = 16384
    q8, sq = M.quantize_e4m3(torch.randn(B, S8, H, D, device=dev))
    k8, sk = M.quantize_e4m3(torch.randn(B, S8, H, D, device=dev))
    v8, sv = M.quantize_e4m3(torch.randn(B, S8, H, D, device=dev))
    o8 = torch.empty(B, S8, H, D, dtype=torch.bfloat16, device=dev)
    l8 = torch.empty(B, H, S8, dtype=torch.float32, device=dev)
    ms = timeit(lambda: M.attn_fwd_block(q8, k8, v8, scale, q_descale=sq, k_descale=sk, v_descale=sv, out=o8, lse=l8),
                n=5, w=2)
    out["fwd_e4m3_16384x16384"] = {"ms": round(ms, 4), "tflops": round(4.0 * B * H * S8 * S8 * D / ms / 1e9, 1),
                                   "pct_of_fp8_mfma_peak": round(4.0 * B * H * S8 * S8 * D / ms / 1e9 / 50.0, 2)}
    # one rank's fp8 step over a 2 x 4 double ring: 8 chunks of 16384 keys, merges included
    chunks8 = [torch.stack([k8, v8]) for _ in range(8)]          # timing only: every rank's chunk has the same bytes
    ms = timeit(lambda: M.fp8_pack_split_kv(q8, chunks8[5], o8, l8, scale, sq, sk, sv,
                                            ring=M.LocalRing((4, 2), 5, chunks8)), n=3, w=1)
    out["step_e4m3_double_ring_16384x8"] = {"ms": round(ms, 3), "tflops": round(8 * 4.0 * B * H * S8 * S8 * D / ms / 1e9, 1)}
    del q8, k8, v8, o8, l8, chunks8
    # one rank's causal GQA step in the zigzag layout: B2, 32 q / 8 kv heads, 2 x 4096 local rows, 8 chunks
    Bz, Hq, Hkv, Sz, W = 2, 32, 8, 8192, 8
    qz = torch.randn(Bz, Sz, Hq, D, device=dev).bfloat16()
    chunks = [torch.randn(2, Bz, Sz, Hkv, D, device=dev).bfloat16() for _ in range(W)]
    oz = torch.empty_like(qz)
    lz = torch.empty(Bz, Hq, Sz, dtype=torch.float32, device=dev)
    ms = timeit(lambda: M.zigzag_causal_pack_kv(qz, chunks[0], oz, lz, scale, ring=M.LocalRing((W,), 0, chunks)),
                n=5, w=2)
    # a diagonal step and each of the 7 other steps cover half of a full 8192 x 8192 block
    flops = (0.5 + 7 * 0.5) * 4.0 * Bz * Hq * Sz * Sz * D
    out["step_bf16_zigzag_causal_gqa_8192x8"] = {"ms": round(ms, 3), "tflops": round(flops / ms / 1e9, 1)}
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-heads", type=int, default=32, help="heads in the CPU baseline sample (0 = skip)")
    ap.add_argument("--sustain", type=float, default=1.5,
                    help="seconds of back-to-back steps for the `sustained` figure (0 = skip)")
    ap.add_argument("--no-variants", action="store_true",
                    help="skip everything after the headline step: the short timings of the causal, backward and "
                         "fp8 block kernels and the low-toggle operand runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one rank's step on ONE GPU (the ring is emulated by local buffer rotation); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    import torch

    import mercury_artifact_amd as M
    from mercury_artifact_amd import flash_attn_interface as FI
    from mercury_artifact_amd import merge as MG

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    B, Sq, H, D, W, rank = 1, 4096, 32, 128, 8, 0
    torch.manual_seed(0)
    q = torch.randn(B, Sq, H, D).bfloat16().to(dev)
    kvs = [torch.randn(2, B, Sq, H, D).bfloat16().to(dev) for _ in range(W)]
    o = torch.empty_like(q)
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device=dev)
    scale = D ** -0.5

    # per-kernel durations: HIP events on the stream the kernels are launched on (torch's current one), inside
    # the timed region.  An event pair costs a few microseconds of stream time, so each step brackets ONE of its
    # forward launches (rotating through the chunks) and the fold; the literal chain further down brackets ONE
    # of its plain merges per step.
    fwd_events, merge_events = [], []
    real_fwd, real_merge = FI.attn_fwd_block, MG.merge_into
    recording = {"on": False, "step": 0, "fwd": 0, "merge": 0}

    def timed(real, bucket, kind, per_step, eligible):
        def wrapper(*a, **kw):
            if not recording["on"] or not eligible(a):
                return real(*a, **kw)
            idx = recording[kind]
            recording[kind] = idx + 1
            if idx != recording["step"] % per_step:
                return real(*a, **kw)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = real(*a, **kw)
            e1.record()
            bucket.append((e0, e1))
            return r
        return wrapper

    FI.attn_fwd_block = timed(real_fwd, fwd_events, "fwd", W, lambda a: True)
    # plain merges only (they run in the literal chain timed further down): the first call is a cast
    MG.merge_into = timed(real_merge, merge_events, "merge", W - 1, lambda a: a[0] is not None and a[4] is not None)

    many_events = []
    real_many = MG.merge_many

    def timed_many(*a, **kw):
        if not recording["on"]:
            return real_many(*a, **kw)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        r = real_many(*a, **kw)
        e1.record()
        many_events.append((e0, e1))
        return r

    from mercury_artifact_amd import ring as RG
    RG.merge_many = timed_many

    def step(literal=False):
        ring = M.LocalRing((W,), rank, kvs)
        M.flash_attn_pack_kv(q, kvs[rank], o, lse, scale, ring=ring, fused_epilogue=not literal,
                             deferred_merge=not literal)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    recording["on"] = True
    t0 = time.perf_counter()
    for i in range(args.steps):
        recording.update(step=i, fwd=0, merge=0)
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    recording["on"] = False

    ms_per_step = dt / args.steps * 1e3
    flops_per_block = 4.0 * B * H * Sq * Sq * D
    # the same step sustained: at least `--sustain` seconds of back-to-back steps (the 20-step window above is
    # 40 ms; the clock the power management settles at shows only after a few hundred milliseconds)
    sustained = None
    if args.sustain > 0:
        n_sus = max(int(args.sustain * 1e3 / ms_per_step) + 1, args.steps)
        s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s0.record()
        for _ in range(n_sus):
            step()
        s1.record()
        smi = smi_snapshot()                      # read while the queued steps run
        torch.cuda.synchronize()
        sus_ms = s0.elapsed_time(s1) / n_sus
        sustained = {"steps": n_sus, "seconds": round(sus_ms * n_sus / 1e3, 3), "ms_per_step": round(sus_ms, 4),
                     "tflops": round(flops_per_block * W / sus_ms / 1e9, 1),
                     "pct_of_bf16_mfma_peak": round(flops_per_block * W / sus_ms / 1e9 / PEAK_BF16_TFLOPS * 100, 2),
                     "amd_smi_during_run": smi}
    flops_per_step = flops_per_block * W
    value = flops_per_step / (ms_per_step * 1e-3) / 1e12

    fwd_ms = sum(e0.elapsed_time(e1) for e0, e1 in fwd_events) / max(len(fwd_events), 1)
    fwd_tflops = flops_per_block / (fwd_ms * 1e-3) / 1e12
    rows = B * Sq * H
    many_bytes = rows * (W * (D * 2 + 4) + D * 2 + 4)
    many_ms = sum(e0.elapsed_time(e1) for e0, e1 in many_events) / max(len(many_events), 1)
    many_gbs = many_bytes / (many_ms * 1e-3) / 1e9

    # the same step as the generated code spells it: update_out_and_lse after every chunk (the fp32
    # accumulator read and written once per chunk), then the cast and the transposed copy of the epilogue.
    # Also timed, with one plain merge per step bracketed by events.
    for _ in range(2):
        step(True)
    torch.cuda.synchronize()
    recording["on"] = True
    t0 = time.perf_counter()
    for i in range(args.steps):
        recording.update(step=i, fwd=W + 1, merge=0)      # forward launches are not sampled again
        step(True)
    torch.cuda.synchronize()
    unfused_ms = (time.perf_counter() - t0) / args.steps * 1e3
    recording["on"] = False
    merge_bytes = rows * (D * 10 + 12)
    real_merges = merge_events
    merge_ms = sum(e0.elapsed_time(e1) for e0, e1 in real_merges) / max(len(real_merges), 1)
    merge_gbs = merge_bytes / (merge_ms * 1e-3) / 1e9
    # what an event pair reads around a kernel that does next to nothing (one element), launched the same way
    # between two other kernels: the part of every bracketed duration above that is not the kernel's own
    # (reported, not subtracted; it matters for the 30 us merge, not for the forward launch)
    one = torch.zeros(1, device=dev)
    tiny = []
    for _ in range(20):
        dst_probe = o.float()                    # some preceding work on the stream
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        one.add_(1.0)
        e1.record()
        tiny.append((e0, e1))
        del dst_probe
    torch.cuda.synchronize()
    tiny_ms = sorted(e0.elapsed_time(e1) for e0, e1 in tiny)[len(tiny) // 2]

    # the drop-in boundary itself: a step function spelled the way the generator spells it (bare names resolved in
    # the exec namespace, update_out_and_lse per chunk, the two epilogue stores), run unchanged in
    # namespace(lazy_merge=True), where the merges of the step are recorded and folded once by the epilogue
    FI.attn_fwd_block, MG.merge_into, RG.merge_many = real_fwd, real_merge, real_many
    drop_in_ms = {}
    for lazy in (False, True):
        ring_box = {}
        ns = {"torch": torch, "WORLD": W, "RANK": rank, "SendRecv": lambda: ring_box["ring"]}
        ns.update(M.namespace(lazy_merge=lazy))
        exec(GENERATED_STEP_TEXT, ns)

        def drop_in_step():
            ring_box["ring"] = M.LocalRing((W,), rank, kvs)
            ns["generated_ring_step"](q, kvs[rank], o, lse, scale)

        for _ in range(2):
            drop_in_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            drop_in_step()
        torch.cuda.synchronize()
        drop_in_ms[lazy] = (time.perf_counter() - t0) / args.steps * 1e3

    # the same step replayed as one HIP graph (one launch instead of ~25; identical kernels and results)
    graph_ms, graph_same = None, None
    try:
        graphed = M.GraphedStep(step)
        eager_o, eager_lse = o.clone(), lse.clone()
        o.zero_()
        graphed.replay()
        torch.cuda.synchronize()
        graph_same = bool(torch.equal(o, eager_o) and torch.equal(lse, eager_lse))
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graphed.replay()
        torch.cuda.synchronize()
        graph_ms = round((time.perf_counter() - t0) / args.steps * 1e3, 4)
    except RuntimeError as exc:      # reported, never fatal for the headline number
        print(f"bench.py: graph replay skipped: {exc}", file=sys.stderr)

    # the same step with every other block launch on a second stream (the driver's two_streams option): the tail
    # of one launch overlaps the head of the next.  Reported next to the headline, not part of it: per-launch
    # durations cannot be bracketed in this mode.
    def step_two_streams():
        M.flash_attn_pack_kv(q, kvs[rank], o, lse, scale, ring=M.LocalRing((W,), rank, kvs), two_streams=True)

    two_streams_ms, two_same = None, None
    if not args.no_variants:                 # overlapping launches would spoil a profiler's per-kernel averages
        for _ in range(3):
            step_two_streams()
        torch.cuda.synchronize()
        two_same = bool(torch.equal(o, eager_o) and torch.equal(lse, eager_lse)) if graph_same is not None else None
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step_two_streams()
        torch.cuda.synchronize()
        two_streams_ms = round((time.perf_counter() - t0) / args.steps * 1e3, 4)

    # one plain streaming kernel of known size (reads 128 MiB of bf16, writes 256 MiB of fp32): the
    # calibration point for the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this script
    calib = torch.empty(64 * 1024 * 1024, dtype=torch.bfloat16, device=dev).normal_()
    MG.grad_accumulate(None, calib)
    torch.cuda.synchronize()
    del calib

    # what a plain device-to-device copy of 256 MiB reaches on this box (read + write bytes over time): the
    # practical ceiling next to the 8 TB/s the merge kernels are priced against
    src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    for _ in range(10):
        dst.copy_(src)
    c1.record()
    torch.cuda.synchronize()
    copy_gbs = 2 * src.numel() * 4 / (c0.elapsed_time(c1) / 10 * 1e-3) / 1e9
    del src, dst

    variants = None if args.no_variants else other_kernels(torch, M, dev)

    props = torch.cuda.get_device_properties(0)
    result = {
        "metric": "per-rank ring-attn step TFLOP/s + % MFMA peak (bf16, d128, Q 4096 x 8 chunks)",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "headline bf16 configuration: non-causal MHA, B1 H32 D128, local Q 4096 x 8 KV chunks "
                               "of 4096 (single ring, rank 0), 8 block forwards + one fold of the 8 block results",
                   "flops_per_step": flops_per_step, "pct_of_bf16_mfma_peak": round(100 * value / PEAK_BF16_TFLOPS, 2),
                   "literal_merge_chain_ms_per_step": round(unfused_ms, 4),
                   "generated_text_ms_per_step": round(drop_in_ms[False], 4),
                   "generated_text_lazy_namespace_ms_per_step": round(drop_in_ms[True], 4),
                   "generated_text_lazy_namespace_tflops": round(flops_per_step / drop_in_ms[True] / 1e9, 1),
                   "hip_graph_ms_per_step": graph_ms, "hip_graph_bit_identical": graph_same,
                   "two_streams_ms_per_step": two_streams_ms, "two_streams_bit_identical": two_same,
                   "device": props.gcnArchName, "cus": props.multi_processor_count,
                   "d2d_copy_gbs": round(copy_gbs, 1)},
        "roofline": {"bound": "mfma", "kernel": "attn_fwd_bf16_d128", "achieved": round(fwd_tflops, 2),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(fwd_tflops / PEAK_BF16_TFLOPS, 4),
                     "traffic": TRAFFIC_FWD_BYTES, "avg_launch_ms": round(fwd_ms, 4), "launches": len(fwd_events)},
        "roofline_merge_many": {"bound": "hbm", "kernel": "lse_merge_many_kernel", "achieved": round(many_gbs, 1),
                                "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(many_gbs / PEAK_HBM_GBS, 4),
                                "traffic": TRAFFIC_MANY_BYTES, "avg_launch_ms": round(many_ms, 5), "launches": len(many_events),
                                "bytes_per_launch": many_bytes},
        "roofline_merge": {"bound": "hbm", "kernel": "lse_merge_kernel", "achieved": round(merge_gbs, 1),
                           "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(merge_gbs / PEAK_HBM_GBS, 4),
                           "traffic": TRAFFIC_MERGE_BYTES, "avg_launch_ms": round(merge_ms, 5), "launches": len(real_merges),
                           "bytes_per_launch": merge_bytes, "event_pair_around_one_element_kernel_ms": round(tiny_ms, 5)},
    }
    result["sustained"] = sustained
    if variants is not None:
        result["forward_kernel_on_low_toggle_operands"] = operand_dependence(torch, M, dev, (B, Sq, H, D), scale)
        result["other_kernels"] = variants
    if args.cpu_heads > 0:
        result["cpu_baseline"] = cpu_baseline(args.cpu_heads, B, Sq, D, W)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
