#!/usr/bin/env python3
"""Benchmark of the paged-KV hot path on one MI355X.

Headline workload (BASELINE.json configs[2], the one the >=70 %-of-HBM target is quoted
on): batched decode, 8 concurrent sequences, contexts U{1024..32768} (seeded, each with a
partially filled last page), f16 K/V, 16 q / 2 kv heads, head_dim 256, 16-token pages on a
60 %-occupied pool whose pages were shuffled and dealt round-robin across the sequences.
A step = append one token per sequence + paged decode attention, for one layer, issued as one
bkv_decode_step call (the attention kernel takes the new row in flight and stores it); layers
rotate so that consecutive steps never touch the same pool bytes.

Prints ONE JSON line.  `value` = algorithmic bytes of a step / wall time of a step, inputs
resident in HBM.  `roofline` prices the split-K attention kernel alone from HIP events on
its stream, attached to each of its dispatches (the kernel's own begin and end).  `cpu_baseline` is the CPU oracle (a restatement of the reference's scalar f64
CPU path) timed on this host on the same workload.  `extra` carries the batch-1 config and
the byte-move kernels.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
N_Q, N_KV, HD, PAGE = 16, 2, 256, 16
ROW_BYTES = N_KV * HD * 2 * 2          # K + V f16 bytes per cell per layer = 2048
# bytes per cell per layer of the quantised pools: f16 K + q8_0 V (36 B per 32 values), and
# int8 K and V with one f16 scale per 32 values (34 B per 32 values)
ROW_BYTES_Q8V = N_KV * (HD * 2 + HD // 32 * 36)   # 1600
ROW_BYTES_I8H = N_KV * 2 * (HD // 32 * 34)        # 1088
# HBM traffic of one launch of the split-K kernel on the default seeded workload, from
# rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this file, each scaled by what the same counter
# reads for the plain copy probe (profiles/hbm_traffic_all_kernels.md)
MEASURED_TRAFFIC = {"seed": 20250003, "fetch_bytes": 329.24e6, "write_bytes": 4.23e6}
APPEND_BYTES_PER_TOKEN = N_KV * HD * (4 + 2) * 2  # f32 in + f16 out, K and V = 6144


def attn_algorithmic_bytes(ctx_after: list[int], row_bytes: int = ROW_BYTES) -> int:
    """K+V rows read once for all heads of a group + block table + q + out."""
    total = 0
    for c in ctx_after:
        total += c * row_bytes + ((c + PAGE - 1) // PAGE) * 4 + 2 * N_Q * HD * 4
    return total


def build_batched(pool_mod, rng, n_seqs: int, lo: int, hi: int, n_layers: int, occupancy: float,
                  layout: int = 0):
    from breccia_amd.kv import Pool

    ctx = []
    for _ in range(n_seqs):
        c = int(rng.integers(lo, hi + 1))
        if c % PAGE == 0:
            c -= 1 + int(rng.integers(0, PAGE - 1))
        ctx.append(c)
    live_pages = sum((c + PAGE) // PAGE + 1 for c in ctx)
    n_pages = int(np.ceil(live_pages / occupancy))
    pool = Pool(n_layers=n_layers, n_pages=n_pages, n_kv_head=N_KV, head_dim=HD, max_seqs=n_seqs + 1,
                max_pages_per_seq=max(ctx) // PAGE + 64, layout=layout)
    pool.set_free_order(rng.permutation(n_pages).astype(np.int32))
    seqs = [pool.seq_create() for _ in ctx]
    # deal the shuffled pages round-robin: one page per sequence per turn
    grown = [0] * n_seqs
    while any(g < c for g, c in zip(grown, ctx)):
        for i, s in enumerate(seqs):
            if grown[i] < ctx[i]:
                grown[i] = min(ctx[i], grown[i] + PAGE)
                pool.seq_reserve(s, grown[i])
    return pool, seqs, ctx


def fill_layers(pool, seqs, ctx, n_layers, rng, stream, keep_host_layer0: bool):
    """N(0,1) f32 K/V through bkv_append, chunked.  Returns layer 0's host K/V per sequence."""
    from breccia_amd.kv import DeviceBuffer

    host = []
    chunk = 4096
    kd = DeviceBuffer(chunk * N_KV * HD * 4)
    vd = DeviceBuffer(chunk * N_KV * HD * 4)
    for i, (s, c) in enumerate(zip(seqs, ctx)):
        k = rng.standard_normal((c, N_KV, HD), dtype=np.float32)
        v = rng.standard_normal((c, N_KV, HD), dtype=np.float32)
        for layer in range(n_layers):
            for at in range(0, c, chunk):
                n = min(chunk, c - at)
                kd.upload(k[at:at + n], stream)
                vd.upload(v[at:at + n], stream)
                pool.append(layer, [s], [at], [n], kd, vd, stream)
                stream.sync()
        host.append((k, v) if keep_host_layer0 else None)
    kd.free()
    vd.free()
    return host


def prepare_steps(pool, seqs, ctx0, n_layers, steps, q_dev, out_dev, newk, newv, stream, first_step=0):
    """Argument blocks of `steps` steps (layer step % n_layers), built ahead of the loop that issues
    them: what a serving loop keeps per batch.  Each item: (layer, positions, ctypes arguments)."""
    import ctypes as C

    n = len(seqs)
    seq_arr = np.ascontiguousarray(seqs, dtype=np.int32)
    ps = seq_arr.ctypes.data_as(C.POINTER(C.c_int32))
    ones = np.ones(n, dtype=np.int32)
    plan = []
    for i in range(first_step, first_step + steps):
        layer, tok = i % n_layers, i // n_layers
        pos = np.ascontiguousarray([c + tok for c in ctx0], dtype=np.int64)
        off = (i % newk.n_slots) * n * N_KV * HD * 4
        plan.append((layer, [int(p) + 1 for p in pos] if layer == 0 else None,
                     pos.ctypes.data_as(C.POINTER(C.c_int64)), newk.at(off), newv.at(off), pos))
    from breccia_amd.kv import PagePair

    return {"plan": plan, "seq_ids": [int(s) for s in seqs], "cow_pairs": (PagePair * 4)(), "n_cow": C.c_int32(),
             "seq_arr": seq_arr, "ps": ps, "ones": ones,
            "pones": ones.ctypes.data_as(C.POINTER(C.c_int32)), "q": q_dev.ptr, "out": out_dev.ptr,
            "stream": stream.handle, "n": n}


def issue_steps(pool, seqs, prep, fused=True):
    """Enqueue the prepared steps: bkv_seq_reserve per sequence when a token begins (layer 0), then one
    bkv_decode_step call per step, or (fused=False) bkv_append followed by bkv_decode_attn."""
    from breccia_amd.kv import check, lib

    n, ps, st, q, out, h = prep["n"], prep["ps"], prep["stream"], prep["q"], prep["out"], pool.handle
    ids, pairs, n_cow = prep["seq_ids"], prep["cow_pairs"], prep["n_cow"]
    reserve, step = lib.bkv_seq_reserve, lib.bkv_decode_step
    for layer, new_lens, pp, k_new, v_new, _pos in prep["plan"]:
        if new_lens is not None:
            for s, new_len in zip(ids, new_lens):
                check(reserve(h, s, new_len, pairs, 4, n_cow))
                if n_cow.value:  # no sequence of this workload shares a page
                    raise RuntimeError("bkv_seq_reserve reported a copy-on-write pair in the bench workload")
        if fused:
            check(step(h, layer, n, ps, pp, k_new, v_new, N_Q, q, None, 0, 0, 1.0 / 16.0, out, st))
        else:
            check(lib.bkv_append(h, layer, n, ps, pp, prep["pones"], k_new, v_new, st))
            check(lib.bkv_decode_attn(h, layer, n, ps, pp, N_Q, q, None, 0, 0, 1.0 / 16.0, out, st))


def run_steps(pool, seqs, ctx0, n_layers, steps, q_dev, out_dev, newk, newv, stream, first_step=0,
              fused=True):
    """Prepare and enqueue `steps` steps (append + attention on layer step % n_layers)."""
    issue_steps(pool, seqs, prepare_steps(pool, seqs, ctx0, n_layers, steps, q_dev, out_dev, newk, newv, stream,
                                          first_step), fused)


def time_steps(pool, seqs, ctx0, n_layers, steps, warmup, bufs, stream, first_step=0, fused=True):
    """(wall milliseconds of `steps` steps between two device-wide synchronisations, the same up to the
    synchronisation of the stream that carries them)."""
    from breccia_amd.kv import Event, device_sync

    q_dev, out_dev, newk, newv = bufs
    run_steps(pool, seqs, ctx0, n_layers, warmup, q_dev, out_dev, newk, newv, stream, first_step, fused)
    prep = prepare_steps(pool, seqs, ctx0, n_layers, steps, q_dev, out_dev, newk, newv, stream, first_step + warmup)
    stream.sync()
    device_sync()
    t0 = time.perf_counter()
    issue_steps(pool, seqs, prep, fused)
    stream.sync()
    stream_ms = (time.perf_counter() - t0) * 1e3
    device_sync()  # nothing else is pending: every launch of the region was on `stream`
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms, stream_ms


def event_steps(pool, seqs, ctx0, n_layers, steps, bufs, stream, first_step):
    """Milliseconds of `steps` steps between two events recorded on the stream."""
    from breccia_amd.kv import Event

    prep = prepare_steps(pool, seqs, ctx0, n_layers, steps, *bufs, stream, first_step)
    e0, e1 = Event(), Event()
    e0.record(stream)
    issue_steps(pool, seqs, prep)
    e1.record(stream)
    stream.sync()
    ms = e0.elapsed_ms(e1)
    e0.close()
    e1.close()
    return ms


def time_replay(pool, seqs, n_layers, tokens, bufs, stream):
    """The same step through a step plan: one token (n_layers x bkv_step_plan_decode + one advance)
    captured into a graph and replayed `tokens` times after a few untimed replays.  Returns
    microseconds per layer.  The sequences go on from their current lengths."""
    from breccia_amd.kv import Graph, StepPlan

    q_dev, out_dev, newk, newv = bufs
    n = len(seqs)
    warm = 4
    pos = [pool.seq_len(s) for s in seqs]
    for s, p in zip(seqs, pos):
        pool.seq_reserve(s, p + tokens + warm + 1)
    plan = StepPlan(pool, seqs, pos, tokens + warm + 1, N_Q, stream=stream)
    g = Graph(stream)
    for layer in range(n_layers):
        off = layer * n * N_KV * HD * 4
        plan.decode(layer, newk.at(off), newv.at(off), q_dev, out_dev, 1.0 / 16.0, stream=stream)
    plan.advance(stream)
    g.end()
    for _ in range(warm):
        g.launch(stream)
    stream.sync()
    t0 = time.perf_counter()
    for _ in range(tokens):
        g.launch(stream)
    stream.sync()
    us = (time.perf_counter() - t0) * 1e6 / (tokens * n_layers)
    _, steps, status = plan.state(stream)
    assert steps == tokens + warm and status == 0, (steps, status)
    g.destroy()
    plan.destroy()
    return us


PREHEAT_MS = 40.0
REGIONS = 5           # timed regions of --steps steps; the median is reported
CPU_SAMPLE_S = 10.0   # CPU time spent on the one-thread baseline


def preheat(pool, seqs, ctx0, n_layers, bufs, stream, ms: float, first_step: int = 0):
    """Run the step for about `ms` milliseconds of wall time (in bursts of 50, synchronised);
    returns (steps run, milliseconds spent).  Not part of the warm-up or of the timed steps."""
    t0 = time.perf_counter()
    done = 0
    while (time.perf_counter() - t0) * 1e3 < ms:
        run_steps(pool, seqs, ctx0, n_layers, 50, *bufs, stream, first_step=first_step + done)
        stream.sync()
        done += 50
    return done, (time.perf_counter() - t0) * 1e3


def make_step_buffers(n_seqs, rng, slots=64):
    from breccia_amd.kv import DeviceBuffer

    q = rng.standard_normal((n_seqs, N_Q, HD), dtype=np.float32)
    q_dev = DeviceBuffer.from_numpy(q)
    out_dev = DeviceBuffer(q.nbytes)
    newk = DeviceBuffer.from_numpy(rng.standard_normal((slots, n_seqs, N_KV, HD), dtype=np.float32))
    newv = DeviceBuffer.from_numpy(rng.standard_normal((slots, n_seqs, N_KV, HD), dtype=np.float32))
    newk.n_slots = newv.n_slots = slots
    return q, (q_dev, out_dev, newk, newv)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-extra", action="store_true", help="skip batch-1 / byte-move extras")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the paged-KV path here is single-device "
              "(--gpus %d is not supported)" % args.gpus, file=sys.stderr)
        return 2

    from breccia_amd import lib as L
    from breccia_amd.kv import DeviceBuffer, Stream, device_info, device_sync, wait_options

    dev_name, n_cu, mem = device_info()
    stream = Stream()
    rng = np.random.Generator(np.random.PCG64(20250003))
    n_layers = 4
    pool, seqs, ctx = build_batched(None, rng, 8, 1024, 32768, n_layers, 0.6)
    host_kv = fill_layers(pool, seqs, ctx, n_layers, rng, stream, keep_host_layer0=not args.no_cpu)
    q_host, bufs = make_step_buffers(len(seqs), rng)

    # ---- clock ramp: the same step, untimed and uncounted, for a fixed wall time -----------
    # (the first tens of milliseconds after the set-up phase run at lower clocks whatever --warmup is)
    pre_steps, pre_ms = preheat(pool, seqs, ctx, n_layers, bufs, stream, PREHEAT_MS)

    # ---- headline: K steps, whole path ------------------------------------------------
    # REGIONS consecutive timed regions of --steps steps each (every one bracketed by host
    # synchronisations); ms_per_step is the median region's, the spread goes into `extra`
    region_ms, region_stream_ms = [], []
    for r in range(REGIONS):
        wall_ms, stream_ms = time_steps(pool, seqs, ctx, n_layers, args.steps, args.warmup if r == 0 else 0, bufs, stream,
                                     first_step=pre_steps + (args.warmup + r * args.steps if r else 0))
        region_ms.append(wall_ms / args.steps)
        region_stream_ms.append(stream_ms / args.steps)
    ms_per_step = float(np.median(region_ms))
    ctx_mid = [c + 1 + (pre_steps + args.warmup + REGIONS * args.steps // 2) // n_layers for c in ctx]
    pre_steps += (REGIONS - 1) * args.steps          # steps taken so far = pre_steps + warmup + steps, as below
    attn_bytes = attn_algorithmic_bytes(ctx_mid)
    step_bytes = attn_bytes + len(seqs) * APPEND_BYTES_PER_TOKEN
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- roofline: the split-K kernel alone, HIP events attached to its dispatches ---------
    pool.timing_reset()
    pool.timing_enable(True)
    first = pre_steps + args.warmup + args.steps
    run_steps(pool, seqs, ctx, n_layers, args.steps, *bufs, stream, first_step=first)
    stream.sync()
    pool.timing_enable(False)
    n_split, ms_split = pool.timing_read(L.STAGE_ATTN_SPLIT)
    n_merge, ms_merge = pool.timing_read(L.STAGE_ATTN_MERGE)
    split_us = ms_split / max(n_split, 1) * 1e3
    # the same steps between two events on the stream (no host time at either end)
    ev_ms = event_steps(pool, seqs, ctx, n_layers, args.steps, bufs, stream, first + args.steps)
    first += args.steps
    # the same steps as two calls (bkv_append, then bkv_decode_attn), for comparison
    two_ms, _ = time_steps(pool, seqs, ctx, n_layers, max(args.steps // 2, 1), 4, bufs, stream,
                           first_step=first + args.steps, fused=False)
    two_call_us = two_ms / max(args.steps // 2, 1) * 1e3
    achieved = attn_bytes / (split_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": MEASURED_TRAFFIC["fetch_bytes"] + MEASURED_TRAFFIC["write_bytes"],
                "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE profile of this command (seed %d), "
                                  "profiles/hbm_traffic_all_kernels.md; a constant of this file, not measured "
                                  "by this run" % MEASURED_TRAFFIC["seed"],
                "kernel": "decode_attn_mfma_kernel<true, false, false> (f16 K/V, all 8 q heads of a kv head per pass on the "
                          "matrix cores, new row taken in flight)",
                "avg_us": round(split_us, 2),
                "launches": n_split, "algorithmic_bytes": attn_bytes}

    # ---- sanity: one sequence of the last step against the oracle ----------------------
    checked = None
    cpu = None
    if not args.no_cpu:
        import oracle

        out = bufs[1].download(np.float32, stream=stream).reshape(len(seqs), N_Q, HD)
        # shortest sequence, layer of the last step
        last = first + args.steps + max(args.steps // 2, 1) + 4 - 1   # `first` counts the preheat steps
        layer = last % n_layers
        i = int(np.argmin(ctx))
        pos = ctx[i] + last // n_layers
        k, v = pool.gather(layer, seqs[i], 0, pos + 1, stream)
        want = oracle.attend(q_host[i], k, v, oracle.dense_cells(pos), pos, N_Q, N_KV, HD, threads=8)
        checked = float(np.max(np.abs(out[i].astype(np.float64) - want)))

        # ---- CPU baseline: the oracle on the same batch (layer 0 contents), one thread -----
        kf = [oracle.to_f16(k) for k, _ in host_kv]
        vf = [oracle.to_f16(v) for _, v in host_kv]
        cells = [oracle.dense_cells(c - 1) for c in ctx]
        # whole steps of the batch, repeated until about CPU_SAMPLE_S seconds of CPU work have been timed
        t0 = time.perf_counter()
        cpu_reps = 0
        while cpu_reps == 0 or (time.perf_counter() - t0 < CPU_SAMPLE_S and cpu_reps < 64):
            for j in range(len(seqs)):
                oracle.attend(q_host[j], kf[j], vf[j], cells[j], ctx[j] - 1, N_Q, N_KV, HD, threads=1)
            cpu_reps += 1
        cpu_total_s = time.perf_counter() - t0
        cpu_s = cpu_total_s / cpu_reps
        cpu_bytes = attn_algorithmic_bytes(ctx)
        nthr = min(oracle.max_threads(), 16)
        t0 = time.perf_counter()
        for _ in range(8):
            for j in range(len(seqs)):
                oracle.attend(q_host[j], kf[j], vf[j], cells[j], ctx[j] - 1, N_Q, N_KV, HD, threads=nthr)
        cpu_mt_s = (time.perf_counter() - t0) / 8
        try:
            affinity = len(os.sched_getaffinity(0))
        except AttributeError:
            affinity = None
        cpu = {"value": round(cpu_bytes / cpu_s / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
               "nproc": os.cpu_count(), "affinity": affinity,
               "sample": "%d full batch-8 decode-attention steps (all 8 sequences, 16 heads, %d cells "
                         "each) in the scalar f64 oracle: %.1f s of CPU time, %.2f s a step"
                         % (cpu_reps, sum(ctx), cpu_total_s, cpu_s),
               "us_per_layer": round(cpu_s * 1e6, 0),
               "openmp": {"threads": nthr, "value": round(cpu_bytes / cpu_mt_s / 1e9, 4),
                          "seconds": round(cpu_mt_s, 3)}}
        del kf, vf, host_kv

    # and as one token (4 layers + advance) captured into a graph and replayed
    replay_us = time_replay(pool, seqs, n_layers, max(args.steps // n_layers, 5), bufs, stream)
    extra = {"attn_split_us": round(split_us, 2), "attn_merge_us": round(ms_merge / max(n_merge, 1) * 1e3, 2),
             "two_call_us_per_layer": round(two_call_us, 2),
             "graph_replay_us_per_layer": round(replay_us, 2),
             "step_event_ms": round(ev_ms / args.steps, 4),
             "timed_regions": {"count": REGIONS, "steps_each": args.steps, "reported": "median",
                               "ms_per_step": [round(x, 5) for x in region_ms],
                               "end_of_region": "bkv_stream_sync of the stream that carries every launch, then bkv_device_sync",
                               "median_ms_per_step_up_to_the_stream_sync": round(float(np.median(region_stream_ms)), 5),
                               "min_ms_per_step": round(min(region_ms), 5), "max_ms_per_step": round(max(region_ms), 5),
                               "frac_of_hbm_peak_min_max": [round(step_bytes / (max(region_ms) * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                                            round(step_bytes / (min(region_ms) * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)]},
             "preheat_ms": round(pre_ms, 1), "preheat_steps": pre_steps,
             "host_wait": {"timed_regions_end_with": "bkv_stream_sync of the bench library: it polls hipStreamQuery "
                                                     "(with a pause instruction) for up to 4 ms before it blocks",
                           "product_wait_options_ms_us": list(wait_options())},
             "contexts": ctx, "pool_pages": pool.desc.n_pages, "device": dev_name, "cus": n_cu,
             "oracle_check_max_abs": checked}
    pool.destroy()
    for b in bufs:
        b.free()

    if not args.no_extra:
        extra.update(bench_batch1(stream, check=not args.no_cpu))
        extra.update(bench_head_counts(stream))
        extra.update(bench_quantised(stream))
        extra.update(bench_select(stream))
        extra.update(bench_prefill(stream))
        extra.update(bench_moves(stream))
        extra.update(bench_prefix_tiers(stream))
        extra.update(bench_reference_cell(stream))
        extra.update(bench_config3_scenario(stream))

    line = {"metric": "paged decode-attn step throughput, batch 8 mixed 1k-32k (append + attention, "
                      "algorithmic bytes / time)",
            "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16 storage, f32 accumulate",
            "data": "synthetic N(0,1), seeded",
            "config": {"workload": "BASELINE configs[2]: batched decode, 8 sequences, ctx U{1k..32k}, "
                                   "f16 KV, 16q/2kv, d256, page 16, 60% occupied shuffled pool; "
                                   "step = append 1 token/seq + paged decode attention, 1 layer (bkv_decode_step)",
                       "layers_rotated": n_layers, "us_per_layer": round(ms_per_step * 1e3, 2),
                       "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4)},
            "roofline": roofline, "cpu_baseline": cpu, "extra": extra}
    print(json.dumps(line))
    return 0


def bench_batch1(stream, check: bool = True) -> dict:
    """BASELINE configs[1]: one sequence at 4096 context, pages scattered over a 64k-page pool,
    12 layers with independent contents; per-layer latency."""
    from breccia_amd import lib as L
    from breccia_amd.kv import Pool

    rng = np.random.Generator(np.random.PCG64(20250002))
    n_layers, ctx = 12, 4096
    pool = Pool(n_layers=n_layers, n_pages=65536, n_kv_head=N_KV, head_dim=HD, max_seqs=2,
                max_pages_per_seq=512)
    pool.set_free_order(rng.permutation(65536).astype(np.int32))
    s = pool.seq_create()
    pool.seq_reserve(s, ctx)
    from breccia_amd.kv import DeviceBuffer
    kd = DeviceBuffer(ctx * N_KV * HD * 4)
    vd = DeviceBuffer(ctx * N_KV * HD * 4)
    for layer in range(n_layers):
        kd.upload(rng.standard_normal((ctx, N_KV, HD), dtype=np.float32), stream)
        vd.upload(rng.standard_normal((ctx, N_KV, HD), dtype=np.float32), stream)
        pool.append(layer, [s], [0], [ctx], kd, vd, stream)
        stream.sync()
    kd.free()
    vd.free()
    q_host, bufs = make_step_buffers(1, rng)
    steps, warm = 600, 60
    wall_ms, ev_ms = time_steps(pool, [s], [ctx], n_layers, steps, warm, bufs, stream)
    pool.timing_reset()
    pool.timing_enable(True)
    run_steps(pool, [s], [ctx], n_layers, steps, *bufs, stream, first_step=steps + warm)
    stream.sync()
    pool.timing_enable(False)
    n_split, ms_split = pool.timing_read(L.STAGE_ATTN_SPLIT)
    n_merge, ms_merge = pool.timing_read(L.STAGE_ATTN_MERGE)
    two_ms, _ = time_steps(pool, [s], [ctx], n_layers, steps // 2, 12, bufs, stream,
                           first_step=2 * steps + warm, fused=False)
    bytes_step = attn_algorithmic_bytes([ctx + 1 + (warm + steps // 2) // n_layers])
    us = wall_ms / steps * 1e3
    checked = None
    if check:
        # the last step's output (two-call form) and the last fused step's, against the oracle
        import oracle

        def against_oracle(step_index):
            layer, pos = step_index % n_layers, ctx + step_index // n_layers
            got = bufs[1].download(np.float32, stream=stream).reshape(N_Q, HD)
            k, v = pool.gather(layer, s, 0, pos + 1, stream)
            want = oracle.attend(q_host[0], k, v, oracle.dense_cells(pos), pos, N_Q, N_KV, HD, threads=8)
            return float(np.max(np.abs(got.astype(np.float64) - want)))

        two_call = against_oracle(2 * steps + warm + steps // 2 + 12 - 1)
        nxt = 2 * steps + warm + steps // 2 + 12
        run_steps(pool, [s], [ctx], n_layers, 1, *bufs, stream, first_step=nxt)
        stream.sync()
        checked = max(two_call, against_oracle(nxt))
    replay_us = time_replay(pool, [s], n_layers, 50, bufs, stream)
    out = {"batch1": {"workload": "BASELINE configs[1]: 1 sequence, ctx 4096, 64k-page pool, 12 layers",
                      "us_per_layer": round(us, 2), "GBps": round(bytes_step / (us * 1e-6) / 1e9, 1),
                      "frac_of_hbm_peak": round(bytes_step / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                      "attn_split_us": round(ms_split / max(n_split, 1) * 1e3, 2),
                      "attn_merge_us": round(ms_merge / max(n_merge, 1) * 1e3, 2),
                      "two_call_us_per_layer": round(two_ms / (steps // 2) * 1e3, 2),
                      "graph_replay_us_per_layer": round(replay_us, 2),
                      "ms_per_token_12_layers": round(us * 12 / 1e3, 4),
                      "oracle_check_max_abs": checked}}
    pool.destroy()
    for b in bufs:
        b.free()
    return out


def bench_quantised(stream) -> dict:
    """Decode attention over the quantised pools: the headline batch on f16 K + q8_0 V, and
    BASELINE configs[4] (16 sequences, ctx U{8192..131072}, int8 K/V with f16 block scales)."""
    from breccia_amd import lib as L
    from breccia_amd.kv import DeviceBuffer

    res = {}
    cases = [("attn_q8v_batch8", L.LAYOUT_Q8V, ROW_BYTES_Q8V, 8, 1024, 32768, 4, 20250003,
              "headline batch on f16 K + q8_0 V", "decode_attn_mfma_q8v_kernel<true>"),
             ("attn_int8_batch16", L.LAYOUT_I8H, ROW_BYTES_I8H, 16, 8192, 131072, 2, 20250005,
              "BASELINE configs[4]: 16 sequences, ctx U{8k..128k}, int8 K/V + f16 scales",
              "decode_attn_mfma_i8h_kernel<true>")]
    for name, layout, row_bytes, n_seqs, lo, hi, n_layers, seed, what, kernel in cases:
        rng = np.random.Generator(np.random.PCG64(seed))
        pool, seqs, ctx = build_batched(None, rng, n_seqs, lo, hi, n_layers, 0.6, layout)
        # contents: one resident block of N(0,1) rows appended at every chunk of every sequence
        chunk = 8192
        kd = DeviceBuffer.from_numpy(rng.standard_normal((chunk, N_KV, HD), dtype=np.float32))
        vd = DeviceBuffer.from_numpy(rng.standard_normal((chunk, N_KV, HD), dtype=np.float32))
        for layer in range(n_layers):
            for s, c in zip(seqs, ctx):
                for at in range(0, c, chunk):
                    pool.append(layer, [s], [at], [min(chunk, c - at)], kd, vd, stream)
            stream.sync()
        kd.free()
        vd.free()
        _, bufs = make_step_buffers(n_seqs, rng, slots=16)
        steps, warm = 40, 8
        # the same untimed clock-ramp phase as the headline's: these kernels are bound by what the SIMDs
        # issue, and the first ~10 ms after set-up run at lower clocks (I8H: 191 us a launch, then 174)
        pre, _ = preheat(pool, seqs, ctx, n_layers, bufs, stream, PREHEAT_MS)
        wall_ms, _ = time_steps(pool, seqs, ctx, n_layers, steps, warm, bufs, stream, first_step=pre, fused=True)
        pool.timing_reset()
        pool.timing_enable(True)
        run_steps(pool, seqs, ctx, n_layers, steps, *bufs, stream, first_step=pre + steps + warm, fused=True)
        stream.sync()
        pool.timing_enable(False)
        n_split, ms_split = pool.timing_read(L.STAGE_ATTN_SPLIT)
        n_merge, ms_merge = pool.timing_read(L.STAGE_ATTN_MERGE)
        b = attn_algorithmic_bytes([c + 1 + (pre + steps + warm) // n_layers for c in ctx], row_bytes)
        split_us = ms_split / max(n_split, 1) * 1e3
        res[name] = {"workload": what, "kernel": kernel, "cells": sum(ctx), "algorithmic_bytes": b,
                     "us_per_layer": round(wall_ms / steps * 1e3, 2),
                     "attn_split_us": round(split_us, 2),
                     "attn_merge_us": round(ms_merge / max(n_merge, 1) * 1e3, 2),
                     "split_GBps": round(b / split_us / 1e3, 1),
                     "split_frac_of_hbm_peak": round(b / split_us / 1e3 / HBM_PEAK_GBPS, 4)}
        pool.destroy()
        for x in bufs:
            x.free()
    return res


def bench_head_counts(stream) -> dict:
    """The headline batch through bkv_decode_attn (no append) at 16 q heads and at the reference
    model's 24: every head of a kv head shares one pass over the K/V rows."""
    from breccia_amd import lib as L
    from breccia_amd.kv import DeviceBuffer

    res = {}
    rng = np.random.Generator(np.random.PCG64(20250003))
    pool, seqs, ctx = build_batched(None, rng, 8, 1024, 32768, 4, 0.6)
    kd = DeviceBuffer.from_numpy(rng.standard_normal((8192, N_KV, HD), dtype=np.float32))
    for layer in range(4):
        for s, c in zip(seqs, ctx):
            for at in range(0, c, 8192):
                pool.append(layer, [s], [at], [min(8192, c - at)], kd, kd, stream)
    stream.sync()
    kd.free()
    pos = [c - 1 for c in ctx]
    b = attn_algorithmic_bytes(ctx)
    for n_q in (16, 24):
        q = DeviceBuffer.from_numpy(rng.standard_normal((8, n_q, HD), dtype=np.float32))
        out = DeviceBuffer(8 * n_q * HD * 4)
        for i in range(200):
            pool.decode_attn(i % 4, seqs, pos, n_q, q, out, 1.0 / 16.0, stream=stream)
        stream.sync()
        pool.timing_reset()
        pool.timing_enable(True)
        for i in range(100):
            pool.decode_attn(i % 4, seqs, pos, n_q, q, out, 1.0 / 16.0, stream=stream)
        stream.sync()
        pool.timing_enable(False)
        n, ms = pool.timing_read(L.STAGE_ATTN_SPLIT)
        us = ms / max(n, 1) * 1e3
        res["%dq" % n_q] = {"attn_split_us": round(us, 2), "split_GBps": round(b / us / 1e3, 1),
                            "frac_of_hbm_peak": round(b / us / 1e3 / HBM_PEAK_GBPS, 4)}
        q.free()
        out.free()
    pool.destroy()
    return {"attn_head_counts_batch8": res}


def bench_select(stream) -> dict:
    """Attention over selection lists, the reference's long-context regime: 8 sequences of
    U{8k..32k} cells, each query attends 512 selected 4-cell blocks + its own block (2052 cells:
    the reference's top-k budget), f16 pool."""
    from breccia_amd import lib as L
    from breccia_amd.kv import DeviceBuffer

    rng = np.random.Generator(np.random.PCG64(20250006))
    n_layers, n_seqs, max_ids = 4, 8, 513
    pool, seqs, ctx = build_batched(None, rng, n_seqs, 8192, 32768, n_layers, 0.6)
    chunk = 8192
    kd = DeviceBuffer.from_numpy(rng.standard_normal((chunk, N_KV, HD), dtype=np.float32))
    vd = DeviceBuffer.from_numpy(rng.standard_normal((chunk, N_KV, HD), dtype=np.float32))
    for layer in range(n_layers):
        for s, c in zip(seqs, ctx):
            for at in range(0, c, chunk):
                pool.append(layer, [s], [at], [min(chunk, c - at)], kd, vd, stream)
        stream.sync()
    kd.free()
    vd.free()
    ids = np.zeros((n_seqs, max_ids), dtype=np.uint32)
    for i, c in enumerate(ctx):
        own = (c - 1) // 4
        ids[i, :512] = rng.choice(own, size=512, replace=False)
        ids[i, 512] = own
    idd = DeviceBuffer.from_numpy(ids)
    cd = DeviceBuffer.from_numpy(np.full(n_seqs, max_ids, dtype=np.uint32))
    q = DeviceBuffer.from_numpy(rng.standard_normal((n_seqs, N_Q, HD), dtype=np.float32))
    out = DeviceBuffer(n_seqs * N_Q * HD * 4)
    pos = [c - 1 for c in ctx]

    def run(n):
        for i in range(n):
            pool.decode_attn_select(i % n_layers, seqs, pos, N_Q, q, out, 1.0 / 16.0, idd, max_ids, cd,
                                    max_ids, stream=stream)

    from breccia_amd.kv import Event
    run(20)
    stream.sync()
    e0, e1 = Event(), Event()
    e0.record(stream)
    run(200)
    e1.record(stream)
    stream.sync()
    us = e0.elapsed_ms(e1) / 200 * 1e3
    e0.close()
    e1.close()
    pool.timing_reset()
    pool.timing_enable(True)
    run(100)
    stream.sync()
    pool.timing_enable(False)
    n_split, ms_split = pool.timing_read(L.STAGE_ATTN_SPLIT)
    n_merge, ms_merge = pool.timing_read(L.STAGE_ATTN_MERGE)
    cells = n_seqs * (max_ids * 4 - 0)
    b = cells * ROW_BYTES + n_seqs * (max_ids * 4 + 2 * N_Q * HD * 4)
    split_us = ms_split / max(n_split, 1) * 1e3
    res = {"attn_select_batch8": {
        "workload": "8 sequences U{8k..32k}, 513 selected blocks (2052 cells) each, f16",
        "algorithmic_bytes": b, "us_per_layer": round(us, 2), "attn_split_us": round(split_us, 2),
        "attn_merge_us": round(ms_merge / max(n_merge, 1) * 1e3, 2),
        "GBps": round(b / us / 1e3, 1), "split_GBps": round(b / split_us / 1e3, 1)}}
    # the selection itself: indexer score of every pooled block (4 heads x 128) + exact top-512
    n_blocks = [c // 4 for c in ctx]
    pooled = [DeviceBuffer.from_numpy(rng.standard_normal((nb, 128), dtype=np.float32)) for nb in n_blocks]
    iq = DeviceBuffer.from_numpy(rng.standard_normal((n_seqs, 4, 128), dtype=np.float32))

    def run_sel(n):
        for _ in range(n):
            pool.select_blocks(pos, iq, pooled, n_blocks, 4, 128, 512, idd, max_ids, cd, max_ids, stream=stream)

    run_sel(5)
    stream.sync()
    e0, e1 = Event(), Event()
    e0.record(stream)
    run_sel(50)
    e1.record(stream)
    stream.sync()
    res["select_blocks_batch8"] = {"blocks_scored": sum(n_blocks), "kept_per_list": 512,
                                   "us": round(e0.elapsed_ms(e1) / 50 * 1e3, 2)}
    e0.close()
    e1.close()
    pool.timing_reset()
    pool.timing_enable(True)
    run_sel(20)
    stream.sync()
    pool.timing_enable(False)
    n_sc, ms_sc = pool.timing_read(L.STAGE_IDX_SCORE)
    n_tk, ms_tk = pool.timing_read(L.STAGE_TOPK)
    res["select_blocks_batch8"]["idx_score_us"] = round(ms_sc / max(n_sc, 1) * 1e3, 2)
    res["select_blocks_batch8"]["topk_us"] = round(ms_tk / max(n_tk, 1) * 1e3, 2)
    for x in [idd, cd, q, out, iq] + pooled:
        x.free()
    pool.destroy()
    return res


def bench_prefill(stream) -> dict:
    """BASELINE configs[3] shape on the MFMA prefill kernel: 4 sequences, 2048-token prefix in the
    cache, a 1024-token chunk each (appended, then attended causally), 16 q / 2 kv heads; on the
    f16 pool and on the two quantised layouts."""
    from breccia_amd import lib as L
    from breccia_amd.kv import DeviceBuffer, Event, Pool

    rng = np.random.Generator(np.random.PCG64(20250007))
    n_seq, before, T = 4, 2048, 1024
    kd = DeviceBuffer.from_numpy(rng.standard_normal((before + T, N_KV, HD), dtype=np.float32))
    vd = DeviceBuffer.from_numpy(rng.standard_normal((before + T, N_KV, HD), dtype=np.float32))
    q = DeviceBuffer.from_numpy(rng.standard_normal((n_seq * T, N_Q, HD), dtype=np.float32))
    out = DeviceBuffer(n_seq * T * N_Q * HD * 4)
    pairs = n_seq * N_Q * sum(before + t + 1 for t in range(T))      # (query row, cell) pairs
    flops = pairs * HD * 4                                           # q.k and p.v, 2 flop per multiply-add
    res = {}
    for name, layout in (("prefill_attn", L.LAYOUT_F16), ("prefill_attn_q8v", L.LAYOUT_Q8V),
                         ("prefill_attn_i8h", L.LAYOUT_I8H)):
        pool = Pool(n_pages=n_seq * ((before + T) // PAGE + 2), max_seqs=n_seq + 1,
                    max_pages_per_seq=(before + T) // PAGE + 2, layout=layout)
        seqs = [pool.seq_create() for _ in range(n_seq)]
        for s in seqs:
            pool.seq_reserve(s, before + T)
            pool.append(0, [s], [0], [before + T], kd, vd, stream)

        def run(n):
            for _ in range(n):
                pool.prefill_attn(0, seqs, [before] * n_seq, [T] * n_seq, N_Q, q, out, 1.0 / 16.0, stream=stream)

        # untimed clock-ramp phase, as for the headline: the steady state is what is reported
        t_pre = time.perf_counter()
        while (time.perf_counter() - t_pre) * 1e3 < PREHEAT_MS:
            run(3)
            stream.sync()
        e0, e1 = Event(), Event()
        e0.record(stream)
        run(10)
        e1.record(stream)
        stream.sync()
        us = e0.elapsed_ms(e1) / 10 * 1e3
        e0.close()
        e1.close()
        pool.timing_reset()
        pool.timing_enable(True)
        run(5)
        stream.sync()
        pool.timing_enable(False)
        n_k, ms_k = pool.timing_read(L.STAGE_PREFILL_ATTN)
        res[name] = {"workload": "BASELINE configs[3] shape: 4 sequences, prefix 2048 + chunk 1024, 16q/2kv",
                     "us": round(us, 1), "kernel_us": round(ms_k / max(n_k, 1) * 1e3, 1),
                     "useful_TFLOPs": round(flops / us / 1e6, 1),
                     "frac_of_f16_mfma_peak": round(flops / us / 1e6 / 2500.0, 4)}
        pool.destroy()
    res["prefill_attn"]["issued_TFLOPs"] = round(2 * flops / res["prefill_attn"]["us"] / 1e6, 1)
    res["prefill_attn"]["note"] = "q and p enter the MFMAs as hi + lo f16, which doubles the issued work"
    for b in (kd, vd, q, out):
        b.free()
    return res


def bench_reference_cell(stream) -> dict:
    """The one cell the reference publishes stage times for (crates/breccia-kernels/src/qsa/bench.rs:28-33,
    numbers docs/phase-4/01-forward-pass.md:4650-4664, RX 6950 XT): one sequence, T = 1, 24 q / 2 kv
    heads, 512 selected blocks + the token's own block = 2051 cells, gate on, f16 and q8_0 V.  Stages
    here: kv-append (T = 1), selection (indexer score over every pooled block + exact top-512), attention
    over the list (split-K + merge, gate applied in the merge), and the three enqueued back to back."""
    from breccia_amd import lib as L
    from breccia_amd.kv import DeviceBuffer, Event, Pool

    n_q, ctx = 24, 16387                 # pos 16386: the own block holds 3 cells -> 512 * 4 + 3 = 2051
    pos, max_ids = ctx - 1, 513
    rng = np.random.Generator(np.random.PCG64(20250011))
    published = {"hardware": "RX 6950 XT (the reference's own GPU; context, not a like-for-like target)",
                 "source": "docs/phase-4/01-forward-pass.md:4650-4664",
                 "kv_append_us": {"f16": 2.11, "q8v": 6.29}, "attn_scores_softmax_us": 1945.1,
                 "attn_apply_gate_us": {"f16": 649.0, "q8v": 622.4}, "layer_total_us": {"f16": 2707.8, "q8v": 2693.9}}
    res = {"workload": "1 sequence at ctx %d, T = 1, 24 q / 2 kv heads, 512 selected blocks + own block = 2051 "
                       "cells, gate on" % ctx, "reference_published": published}
    rows = DeviceBuffer.from_numpy(rng.standard_normal((ctx, N_KV, HD), dtype=np.float32))
    new = DeviceBuffer.from_numpy(rng.standard_normal((1, N_KV, HD), dtype=np.float32))
    q = DeviceBuffer.from_numpy(rng.standard_normal((1, n_q, HD), dtype=np.float32))
    gate = DeviceBuffer.from_numpy(rng.standard_normal((1, n_q, HD), dtype=np.float32))
    out = DeviceBuffer(n_q * HD * 4)
    n_blocks = pos // 4
    pooled = DeviceBuffer.from_numpy(rng.standard_normal((n_blocks, 128), dtype=np.float32))
    iq = DeviceBuffer.from_numpy(rng.standard_normal((1, 4, 128), dtype=np.float32))
    ids = DeviceBuffer(max_ids * 4)
    cnt = DeviceBuffer(16)

    def timed(fn, reps=200):
        for _ in range(20):
            fn()
        stream.sync()
        e0, e1 = Event(), Event()
        e0.record(stream)
        for _ in range(reps):
            fn()
        e1.record(stream)
        stream.sync()
        us = e0.elapsed_ms(e1) / reps * 1e3
        e0.close()
        e1.close()
        return round(us, 2)

    for tag, layout in (("f16", L.LAYOUT_F16), ("q8v", L.LAYOUT_Q8V)):
        pool = Pool(n_layers=1, n_pages=ctx // PAGE + 64, n_kv_head=N_KV, head_dim=HD, max_seqs=2,
                    max_pages_per_seq=ctx // PAGE + 8, layout=layout)
        pool.set_free_order(rng.permutation(ctx // PAGE + 64).astype(np.int32))
        s = pool.seq_create()
        pool.seq_reserve(s, ctx)
        pool.append(0, [s], [0], [ctx], rows, rows, stream)
        stream.sync()

        def append():
            pool.append(0, [s], [pos], [1], new, new, stream)

        def select():
            pool.select_blocks([pos], iq, [pooled], [n_blocks], 4, 128, 512, ids, max_ids, cnt, max_ids, stream=stream)

        def attend():
            pool.decode_attn_select(0, [s], [pos], n_q, q, out, 1.0 / 16.0, ids, max_ids, cnt, max_ids,
                                    gate_dev=gate, gate_seq_stride=n_q * HD, gate_head_stride=HD, stream=stream)

        def layer():
            append()
            select()
            attend()

        select()
        stream.sync()
        n_sel = int(cnt.download(np.uint32, 1, stream)[0])
        r = {"selected_blocks": n_sel, "kv_append_us": timed(append), "select_us": timed(select),
             "attn_over_list_us": timed(attend), "layer_total_us": timed(layer)}
        pool.timing_reset()
        pool.timing_enable(True)
        for _ in range(50):
            layer()
        stream.sync()
        pool.timing_enable(False)
        for name, stage in (("append", L.STAGE_APPEND), ("idx_score", L.STAGE_IDX_SCORE), ("topk", L.STAGE_TOPK),
                            ("attn_split", L.STAGE_ATTN_SPLIT), ("attn_merge", L.STAGE_ATTN_MERGE)):
            n_k, ms_k = pool.timing_read(stage)
            r[name + "_kernel_us"] = round(ms_k / max(n_k, 1) * 1e3, 2)
        res[tag] = r
        pool.destroy()
    for b in (rows, new, q, gate, out, pooled, iq, ids, cnt):
        b.free()
    return {"reference_cell": res}


def bench_config3_scenario(stream) -> dict:
    """BASELINE configs[3] as worded, timed end to end on one pool: four sequences share a 2040-token
    prefix (127 full pages + a partial one) through refcounts; each appends a distinct 1024-token chunk of
    binary16 K/V (bkv_append_f16), which costs the writers that still share the partial page one
    copy-on-write page copy each; then a seeded 25 % of the pages in use go to pinned host memory and come
    back.  12 layers (the model's full-attention layers), so that a page is 12 x 32 KiB.  At these sizes the
    append and the copies are launch-bound; the bulk legs of bench_moves price the kernels."""
    from breccia_amd.kv import DeviceBuffer, Event, Pool

    rng = np.random.Generator(np.random.PCG64(20250004))
    n_layers, prefix, chunk, n_pages = 12, 2040, 1024, 1024
    pool = Pool(n_layers=n_layers, n_pages=n_pages, n_kv_head=N_KV, head_dim=HD, max_seqs=8,
                max_pages_per_seq=(prefix + chunk) // PAGE + 4)
    pool.set_free_order(rng.permutation(n_pages).astype(np.int32))
    k16 = DeviceBuffer.from_numpy(rng.standard_normal((prefix + 4 * chunk, N_KV, HD), dtype=np.float32).astype(np.float16))
    v16 = DeviceBuffer.from_numpy(rng.standard_normal((prefix + 4 * chunk, N_KV, HD), dtype=np.float32).astype(np.float16))
    row = N_KV * HD * 2
    root = pool.seq_create()
    pool.seq_reserve(root, prefix)
    for layer in range(n_layers):
        pool.append(0 + layer, [root], [0], [prefix], k16, v16, stream, f16_rows=True)
    seqs = [root] + [pool.seq_fork(root, prefix) for _ in range(3)]
    stream.sync()
    e = [Event() for _ in range(4)]
    pairs_all = [pool.seq_reserve(s, prefix + chunk) for s in seqs]
    # copy-on-write copies (all layers of a page in one call), then the four chunks, layer by layer
    e[0].record(stream)
    for pairs in pairs_all:
        pool.page_copy(pairs, stream)
    e[1].record(stream)
    for layer in range(n_layers):
        for i, s in enumerate(seqs):
            off = (prefix + i * chunk) * row
            pool.append(layer, [s], [prefix], [chunk], k16.at(off), v16.at(off), stream, f16_rows=True)
    e[2].record(stream)
    stream.sync()
    n_copies = sum(len(p) for p in pairs_all)
    copy_ms, append_ms = e[0].elapsed_ms(e[1]), e[1].elapsed_ms(e[2])
    used = np.unique(np.concatenate([pool.block_table(s) for s in seqs]))
    cold = rng.choice(used, size=used.size // 4, replace=False).astype(np.int32)
    slab = pool.swap_page_bytes()
    host = pool.host_alloc(cold.size * slab)
    pool.swap_out(cold[:8], host, stream)       # the staging halves' and the side stream's one-time costs
    pool.swap_wait()
    t0 = time.perf_counter()
    pool.swap_out(cold, host, stream)
    pool.swap_wait()
    t_out = time.perf_counter() - t0
    t0 = time.perf_counter()
    pool.swap_in(cold, host, stream)
    pool.swap_fence(stream)
    stream.sync()
    t_in = time.perf_counter() - t0
    app_bytes = 4 * chunk * n_layers * N_KV * HD * (2 + 2) * 2
    copy_bytes = n_copies * n_layers * 2 * 32768
    res = {"workload": "BASELINE configs[3]: 4 sequences on a shared 2040-token prefix, 1024-token f16 chunks "
                       "(bkv_append_f16), copy-on-write of the partial page, 25 % of pages out and back; 12 layers",
           "cow_copies": n_copies, "cow_copy_us_each": round(copy_ms * 1e3 / max(n_copies, 1), 2),
           "cow_copy_GBps": round(copy_bytes / max(copy_ms, 1e-9) / 1e6, 1),
           "append_calls": 4 * n_layers, "append_us_per_call": round(append_ms * 1e3 / (4 * n_layers), 2),
           "append_GBps": round(app_bytes / append_ms / 1e6, 1),
           "swap_pages": int(cold.size), "swap_bytes": int(cold.size * slab),
           "swap_out_GBps": round(cold.size * slab / t_out / 1e9, 2),
           "swap_in_GBps": round(cold.size * slab / t_in / 1e9, 2)}
    host.free()
    for x in e:
        x.close()
    k16.free()
    v16.free()
    pool.destroy()
    return {"config3_scenario": res}


def bench_prefix_tiers(stream) -> dict:
    """The prefix tree's lower tiers: 2048 cached pages (a 32k-token prefix, 64 MiB at one layer)
    demoted to pinned host memory and promoted back by an adopting request; then the same with a
    host arena of 256 pages, so that most pages go on to a file under the temporary directory
    (page cache included: the file is not opened for direct I/O)."""
    import tempfile

    from breccia_amd.kv import DeviceBuffer, Pool

    rng = np.random.Generator(np.random.PCG64(20250008))
    n = 2048
    tokens = rng.integers(0, 32000, size=n * PAGE).astype(np.int32)
    pool = Pool(n_layers=1, n_pages=2 * n + 64, n_kv_head=N_KV, head_dim=HD, max_seqs=4,
                max_pages_per_seq=n + 8)
    slab = pool.swap_page_bytes()
    rows = DeviceBuffer.from_numpy(rng.standard_normal((n * PAGE, N_KV, HD), dtype=np.float32))
    res = {}
    with tempfile.TemporaryDirectory() as tmp:
        for name, host_pages, disk_pages in (("host", n, 0), ("host256_then_file", 256, n)):
            pool.prefix_tiers(host_pages * slab, os.path.join(tmp, "tier3.bin") if disk_pages else None,
                              disk_pages * slab)
            s = pool.seq_create()
            pool.seq_reserve(s, n * PAGE)
            pool.append(0, [s], [0], [n * PAGE], rows, rows, stream)
            stream.sync()
            pool.prefix_insert(s, tokens)
            pool.seq_free(s)
            t0 = time.perf_counter()
            freed = pool.prefix_evict(n)
            pool.swap_wait()
            t_out = time.perf_counter() - t0
            t0 = time.perf_counter()
            s, matched = pool.seq_create_from_prefix(tokens)
            pool.swap_wait()
            t_in = time.perf_counter() - t0
            assert freed == n and matched == n * PAGE
            res[name] = {"pages": n, "bytes": n * slab, "demote_GBps": round(n * slab / t_out / 1e9, 2),
                         "promote_GBps": round(n * slab / t_in / 1e9, 2)}
            pool.seq_free(s)
            pool.prefix_clear()
    rows.free()
    pool.destroy()
    return {"prefix_tiers": res}


def bench_moves(stream) -> dict:
    """Bulk shapes of the byte-move kernels: append (f32 in -> f16 out), copy-on-write page
    copy, VRAM <-> pinned host swap, and a plain device copy for reference."""
    from breccia_amd import lib as L
    from breccia_amd.kv import DeviceBuffer, Event, Pool, check, lib

    rng = np.random.Generator(np.random.PCG64(20250004))
    n_pages = 40960
    pool = Pool(n_layers=1, n_pages=n_pages, n_kv_head=N_KV, head_dim=HD, max_seqs=8,
                max_pages_per_seq=n_pages // 4 + 8)
    assert n_pages >= 2 * 16384
    pool.set_free_order(rng.permutation(n_pages).astype(np.int32))
    res = {}

    def timed(fn, reps):
        fn()
        stream.sync()
        e0, e1 = Event(), Event()
        e0.record(stream)
        for _ in range(reps):
            fn()
        e1.record(stream)
        stream.sync()
        ms = e0.elapsed_ms(e1) / reps
        e0.close()
        e1.close()
        return ms

    # append: 4 sequences x 16384 tokens in one call (BASELINE configs[3] shape, scaled up)
    T = 16384
    seqs = [pool.seq_create() for _ in range(4)]
    for s in seqs:
        pool.seq_reserve(s, 4 * T)   # 4096 pages each: sources for the page-copy leg below
    kd = DeviceBuffer.from_numpy(rng.standard_normal((4 * T, N_KV, HD), dtype=np.float32))
    vd = DeviceBuffer.from_numpy(rng.standard_normal((4 * T, N_KV, HD), dtype=np.float32))
    ms = timed(lambda: pool.append(0, seqs, [0] * 4, [T] * 4, kd, vd, stream), 20)
    b = 4 * T * APPEND_BYTES_PER_TOKEN
    res["append_bulk"] = {"tokens": 4 * T, "ms": round(ms, 4), "GBps": round(b / ms / 1e6, 1),
                          "frac_of_hbm_peak": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    ms = timed(lambda: pool.append(0, seqs, [7] * 4, [1] * 4, kd, vd, stream), 200)
    res["append_decode_us"] = round(ms * 1e3, 2)
    # the same rows handed over as raw f16 (bkv_append_f16): 2048 B in + 2048 B out per token
    ms = timed(lambda: pool.append(0, seqs, [0] * 4, [T] * 4, kd, vd, stream, f16_rows=True), 20)
    b = 4 * T * N_KV * HD * (2 + 2) * 2
    res["append_bulk_f16_rows"] = {"tokens": 4 * T, "ms": round(ms, 4), "GBps": round(b / ms / 1e6, 1),
                                   "frac_of_hbm_peak": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    # K preparation fused into the append (RMSNorm * gamma -> rotary -> store): same bytes
    from breccia_amd.kv import rope_table
    gd = DeviceBuffer.from_numpy(np.ones(HD, dtype=np.float32))
    td = DeviceBuffer.from_numpy(rope_table(1e7, 64, T))
    ms = timed(lambda: pool.append_kprep(0, seqs, [0] * 4, [T] * 4, kd, vd, gd, 1e-6, td, 64, T,
                                         stream=stream), 20)
    b = 4 * T * APPEND_BYTES_PER_TOKEN
    res["append_kprep_bulk"] = {"tokens": 4 * T, "ms": round(ms, 4), "GBps": round(b / ms / 1e6, 1),
                                "frac_of_hbm_peak": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    ms = timed(lambda: pool.append_kprep(0, seqs, [7] * 4, [1] * 4, kd, vd, gd, 1e-6, td, 64, T,
                                         stream=stream), 200)
    res["append_kprep_decode_us"] = round(ms * 1e3, 2)
    pool.timing_reset()
    pool.timing_enable(True)
    for _ in range(5):
        pool.append_kprep(0, seqs, [0] * 4, [T] * 4, kd, vd, gd, 1e-6, td, 64, T, stream=stream)
    stream.sync()
    pool.timing_enable(False)
    n_k, ms_k = pool.timing_read(L.STAGE_APPEND_KPREP)
    res["append_kprep_bulk"]["kernel_ms"] = round(ms_k / max(n_k, 1), 4)
    # the quantised layouts on the same bulk shape: f32 rows in, and raw f16 rows in (BASELINE
    # configs[4]: "quantized from N(0,1) f16 on append")
    k16 = DeviceBuffer.from_numpy(rng.standard_normal((4 * T, N_KV, HD), dtype=np.float32).astype(np.float16))
    v16 = DeviceBuffer.from_numpy(rng.standard_normal((4 * T, N_KV, HD), dtype=np.float32).astype(np.float16))
    for tag, layout, out_bytes in (("q8v", L.LAYOUT_Q8V, ROW_BYTES_Q8V), ("i8h", L.LAYOUT_I8H, ROW_BYTES_I8H)):
        qp = Pool(n_layers=1, n_pages=4 * T // PAGE + 8, n_kv_head=N_KV, head_dim=HD, max_seqs=8,
                  max_pages_per_seq=T // PAGE + 8, layout=layout)
        qp.set_free_order(rng.permutation(4 * T // PAGE + 8).astype(np.int32))
        qs = [qp.seq_create() for _ in range(4)]
        for s in qs:
            qp.seq_reserve(s, T)
        for name, f16_rows, in_bytes in (("append_bulk_" + tag, False, N_KV * HD * 4 * 2),
                                         ("append_bulk_%s_f16_rows" % tag, True, N_KV * HD * 2 * 2)):
            ks, vs = (k16, v16) if f16_rows else (kd, vd)
            ms = timed(lambda: qp.append(0, qs, [0] * 4, [T] * 4, ks, vs, stream, f16_rows=f16_rows), 20)
            b = 4 * T * (in_bytes + out_bytes)
            res[name] = {"tokens": 4 * T, "bytes_per_token": in_bytes + out_bytes, "ms": round(ms, 4),
                         "GBps": round(b / ms / 1e6, 1), "frac_of_hbm_peak": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        ms = timed(lambda: qp.append(0, qs, [7] * 4, [1] * 4, kd, vd, stream), 200)
        res["append_decode_%s_us" % tag] = round(ms * 1e3, 2)
        ms = timed(lambda: qp.append_kprep(0, qs, [0] * 4, [T] * 4, kd, vd, gd, 1e-6, td, 64, T, stream=stream), 20)
        b = 4 * T * (N_KV * HD * 4 * 2 + out_bytes)
        res["append_kprep_bulk_" + tag] = {"tokens": 4 * T, "ms": round(ms, 4), "GBps": round(b / ms / 1e6, 1),
                                           "frac_of_hbm_peak": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        qp.destroy()
    for x in (kd, vd, k16, v16, gd, td):
        x.free()

    # page copy: 16384 pairs = 512 MiB read + 512 MiB written
    used = np.concatenate([pool.block_table(s) for s in seqs])
    free = np.setdiff1d(np.arange(n_pages, dtype=np.int32), used)
    n_pairs = 16384
    pairs = np.stack([used[:n_pairs], free[:n_pairs]], axis=1).astype(np.int32)
    # kernel time from the library's per-kernel events (two launches of 8192 pairs per call);
    # the host-side upload of the 128 KiB pair list is not part of the copy
    pool.page_copy(pairs, stream)
    stream.sync()
    pool.timing_reset()
    pool.timing_enable(True)
    for _ in range(10):
        pool.page_copy(pairs, stream)
    stream.sync()
    pool.timing_enable(False)
    n_l, ms_l = pool.timing_read(L.STAGE_PAGE_COPY)
    ms = ms_l / 10
    b = 2 * n_pairs * 32768
    res["page_copy_bulk"] = {"pairs": n_pairs, "launches_per_call": n_l // 10, "ms": round(ms, 4),
                             "GBps": round(b / ms / 1e6, 1),
                             "frac_of_hbm_peak": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    ms = timed(lambda: pool.page_copy(pairs[:1], stream), 200)
    res["page_copy_one_us"] = round(ms * 1e3, 2)

    # swap: 25 % of the live pages out to pinned host and back
    n_swap = 4096
    host = pool.host_alloc(n_swap * pool.swap_page_bytes())
    pages = used[:n_swap].astype(np.int32)
    # once untimed: the first pass through the staging halves and the side stream pays one-time costs
    pool.swap_out(pages, host, stream)
    pool.swap_wait()
    pool.swap_in(pages, host, stream)
    pool.swap_fence(stream)
    stream.sync()
    t0 = time.perf_counter()
    pool.swap_out(pages, host, stream)
    pool.swap_wait()
    t_out = time.perf_counter() - t0
    t0 = time.perf_counter()
    pool.swap_in(pages, host, stream)
    pool.swap_fence(stream)
    stream.sync()
    t_in = time.perf_counter() - t0
    b = n_swap * pool.swap_page_bytes()
    res["swap"] = {"pages": n_swap, "bytes": b, "out_GBps": round(b / t_out / 1e9, 2),
                   "in_GBps": round(b / t_in / 1e9, 2)}
    # the device-side gather / scatter of the same pages (page_stage_kernel), by the stage timer
    pool.timing_reset()
    pool.timing_enable(True)
    pool.swap_out(pages, host, stream)
    pool.swap_wait()
    pool.timing_enable(False)
    n_ps, ms_ps = pool.timing_read(L.STAGE_PAGE_STAGE)
    res["swap"]["page_stage_launches"] = n_ps
    res["swap"]["page_stage_GBps"] = round(2 * b / max(ms_ps, 1e-9) / 1e6, 1)
    host.free()

    # plain device copy of the same volume (ceiling of a read+write stream on this box); after the
    # swap, because for some tens of milliseconds after large device buffers are freed
    # device-to-host copies run at half their rate
    a = DeviceBuffer(512 << 20)
    c = DeviceBuffer(512 << 20)
    ms = timed(lambda: check(lib.bkv_copy_probe(c.ptr, a.ptr, 512 << 20, stream.handle)), 10)
    res["device_copy_probe"] = {"bytes_moved": 2 * (512 << 20), "ms": round(ms, 4),
                                "GBps": round(2 * (512 << 20) / ms / 1e6, 1)}
    # read-only stream of the same buffer: in address order, and as 8 KiB chunks in a scattered order
    # (what a shuffled pool looks like to the attention kernels) -- the ceiling a read-only kernel
    # can be held against on this box
    sink = DeviceBuffer(16)
    for name, scattered in (("device_read_probe_linear", 0), ("device_read_probe_scattered", 1),
                            ("device_read_probe_scattered_via_lds_loads", 2)):
        ms = timed(lambda: check(lib.bkv_read_probe(a.ptr, 512 << 20, scattered, sink.ptr, stream.handle)), 20)
        res[name] = {"bytes_read": 512 << 20, "ms": round(ms, 4), "GBps": round((512 << 20) / ms / 1e6, 1),
                     "frac_of_hbm_peak": round((512 << 20) / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    sink.free()
    a.free()
    c.free()

    pool.destroy()
    return res


if __name__ == "__main__":
    sys.exit(main())
