#!/usr/bin/env python3
"""Benchmark of the BDH decode state step on one MI355X.

Workload (BASELINE config 2, the configuration the metric is quoted on): one layer's
recurrent state step — RoPE at a position t ~ U[0,4096), readout with the old state and
rank-1 update — on rho f32 [B=32, h=4, N=8192, d=256] (1 GiB), x = relu(N(mu,1)) with
mu = Phi^-1(0.05) (about 5 % active neurons), v ~ N(0,1).  One "step" is one call of
bdh_state_step over the whole batch (32 tokens).  Inputs are resident in HBM before the
timed region; a ring of distinct (x, v) sets keeps caches from helping.

Prints ONE JSON line (see --help for the knobs).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def cpu_baseline(B, h, N, d, freqs, budget_s=12.0, max_steps=20):
    """The restated reference CPU path (dense op sequence of src/model/bdh.rs:288-302 plus the
    rotate), timed on this host on a bounded number of steps of the same workload."""
    from oracle.bdh_oracle import COracle

    orc = COracle()
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    rng = np.random.default_rng(1)
    rho = (0.01 * rng.standard_normal((B, h, N, d), dtype=np.float32))
    x = np.maximum(rng.standard_normal((B, h, N), dtype=np.float32) - np.float32(1.6449), 0)
    v = rng.standard_normal((B, d), dtype=np.float32)
    orc.state_step_dense(x, v, freqs, 17, rho)  # warm-up (page faults, thread pool)
    steps, t0 = 0, time.perf_counter()
    while steps < max_steps and (time.perf_counter() - t0) < budget_s:
        orc.state_step_dense(x, v, freqs, 100 + steps, rho)
        steps += 1
    dt = time.perf_counter() - t0
    one = None
    try:  # the same step on one thread (Burn's ndarray backend threads only its GEMMs)
        import ctypes

        gomp = ctypes.CDLL("libgomp.so.1")
        gomp.omp_set_num_threads(1)
        t1 = time.perf_counter()
        n1 = 0
        while n1 < 3 and (time.perf_counter() - t1) < 6.0:
            orc.state_step_dense(x, v, freqs, 200 + n1, rho)
            n1 += 1
        one = B * n1 / (time.perf_counter() - t1)
        gomp.omp_set_num_threads(threads)
    except OSError:
        pass
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "")
    except OSError:
        pass
    return {
        "value": B * steps / dt,
        "unit": "tokens/s",
        "cores": min(threads, B * h),
        "kind": "port",
        "sample": f"{steps} dense steps of the same config-2 shape (rho f32 [{B},{h},{N},{d}]), "
                  f"C restatement of the reference op sequence (not a Burn binary), OpenMP over (b,h) slices, "
                  f"{dt / steps * 1e3:.1f} ms/step"
                  + (f"; on one thread {one:.0f} tokens/s" if one else "") + (f"; host CPU: {model}" if model else ""),
        "value_one_thread": one,
    }


def cpu_baseline_model(cfg, B, prompt, budget_s=20.0, max_tokens=256):
    """Config 1 end to end on this host with the restated reference path (dense state passes of
    src/model/bdh.rs:288-302, the same seeded weights and prompt as the GPU run): the prompt as
    one call, then greedy decode tokens until the time budget is used."""
    from oracle import bdh_oracle as orc

    c = orc.COracle()
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    shape = orc.BDHShape(n_layer=cfg.n_layer, n_embd=cfg.n_embd, n_head=cfg.n_head,
                         mlp_internal_dim_multiplier=cfg.mlp_internal_dim_multiplier, vocab_size=cfg.vocab_size,
                         rotary=orc.ROPE)
    w = orc.init_weights(shape, 7)
    rho = np.zeros((cfg.n_layer, B, cfg.n_head, shape.latent_per_head, cfg.n_embd), np.float32)
    t0 = time.perf_counter()
    logits, pos, _, _ = c.forward_with_state(shape, w, prompt, rho, 0, sparse_state=False)
    t_prompt = time.perf_counter() - t0
    toks = np.array([[c.greedy_token(logits[b, -1])] for b in range(B)])
    n, t1 = 0, time.perf_counter()
    while n < max_tokens and (time.perf_counter() - t1) < budget_s:
        logits, pos, _, _ = c.forward_with_state(shape, w, toks, rho, pos, sparse_state=False)
        toks = np.array([[c.greedy_token(logits[b, -1])] for b in range(B)])
        n += 1
    dt = time.perf_counter() - t1
    return {"value": B * n / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"{prompt.shape[1]}-token prompt in {t_prompt:.2f} s, then {n} greedy decode tokens at "
                      f"{dt / n * 1e3:.1f} ms/token; C restatement of the reference op sequence with dense state passes, "
                      f"OpenMP; same seeded weights and prompt as the GPU run"}


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


def measure_prefill(B=8, h=4, N=8192, d=256, T=2048, density=0.05, steps=10, warmup=3, rotary="rope",
                    row_normalize=False, all_scores=False):
    """BASELINE config 3: chunked prefill, B=8, T=2048, h=4, N=8192, d=256, bf16 inputs, f32
    accumulate, 5 % density, positions 0..T, fresh state.  One step = one bdh_prefill_chunked (RoPE), or one
    bdh_prefill_chunked_ex for PoPE (2N state rows), ALiBi (decaying state, default slopes) and the row-normalised
    stateless form (time blocks of 64; ALiBi then adds its term to the scores).
    Returns (ms per call, algorithmic FLOP per call)."""
    import torch
    from scipy.stats import norm

    from burn_dragon_amd.kernel.linear_attention import build_freqs
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import prefill_chunked, prefill_chunked_ex

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(4)
    mu = float(norm.ppf(density))
    x = torch.empty((B, h, T, N), device=dev, dtype=torch.bfloat16)
    for b in range(B):  # generated per batch entry to bound the f32 temporary
        x[b] = torch.relu(torch.randn((h, T, N), device=dev, generator=g) + mu).to(torch.bfloat16)
    v = torch.randn((B, T, d), device=dev, generator=g).to(torch.bfloat16)
    rot = RotaryEmbedding.parse(rotary)
    nq = 2 * N if rot == RotaryEmbedding.POPE else N
    freqs = build_freqs(N, 65536.0, rot).reshape(-1).to(dev)
    rho = None if row_normalize else torch.zeros((B, h, nq, d), device=dev)
    if rot == RotaryEmbedding.ROPE and not row_normalize:
        call = lambda: prefill_chunked(x, v, rho, freqs, 0, state_is_zero=True, all_scores=all_scores)
    else:
        slopes = None
        if rot == RotaryEmbedding.ALIBI and row_normalize:  # the additive term needs explicit slopes
            slopes = [1.0 / 2.0 ** (i / h) for i in range(h)]
        call = lambda: prefill_chunked_ex(x, v, rho, freqs, 0, rotary=rot, alibi_slopes=slopes,
                                          row_normalize=row_normalize, block_size=64, state_is_zero=True)
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        call()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = max(start.elapsed_time(stop), wall * 1e3) / steps
    flop = float(B * h) * (T * (T - 1.0) * nq + T * (T - 1.0) * d + (0.0 if row_normalize else 2.0 * T * nq * d))
    return ms, flop


def measure_prefill_queued(B=8, h=4, N=8192, d=256, T=2048, density=0.05, rounds=12, warmup=12):
    """The same work as measure_prefill fed as a queue: two contexts on two streams, each given half-batch calls back
    to back, so the write-bound first kernel of one call runs beside the read-bound second kernel of the other.  A
    throughput figure for servers with independent prompts, not the latency of one call.  Returns ms per B sequences."""
    import torch
    from scipy.stats import norm

    from burn_dragon_amd import ffi
    from burn_dragon_amd.kernel.linear_attention import build_freqs
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import prefill_chunked

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(5)
    mu = float(norm.ppf(density))
    freqs = build_freqs(N, 65536.0, RotaryEmbedding.ROPE).reshape(-1).to(dev)
    half = B // 2
    sets = []
    for _ in range(2):
        x = torch.empty((half, h, T, N), device=dev, dtype=torch.bfloat16)
        for b in range(half):
            x[b] = torch.relu(torch.randn((h, T, N), device=dev, generator=g) + mu).to(torch.bfloat16)
        sets.append((x, torch.randn((half, T, d), device=dev, generator=g).to(torch.bfloat16),
                     torch.zeros((half, h, N, d), device=dev)))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ctxs = [ffi.Context(0, st.cuda_stream) for st in streams]
    torch.cuda.synchronize()

    def one_round():
        for (x, v, rho), st, ctx in zip(sets, streams, ctxs):
            with torch.cuda.stream(st):
                prefill_chunked(x, v, rho, freqs, 0, state_is_zero=True, ctx=ctx)

    for _ in range(warmup):
        one_round()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(rounds):
        one_round()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / rounds
    for ctx in ctxs:
        ctx.close()
    return ms


def prefill_executed_flop(B, h, N, d, T):
    """Matrix-core FLOP the chunk-recurrent form executes (d = 256, N % 256 == 0, T % 256 == 0): per 256-token chunk a
    full 256x256 score tile (K = N), scores x V (K = 256, half of it for the upper row block), the state term
    (K = N, absent for the first chunk of a fresh state) and the state update."""
    nc = T // 256
    per_slice = nc * 2.0 * 256 * 256 * N + nc * 2.0 * 256 * 256 * 192 + (nc - 1) * 2.0 * 256 * d * N + 2.0 * T * N * d
    return B * h * per_slice


def prefill_traffic_bytes(B, h, N, d, T):
    """HBM bytes one call of the chunk-recurrent form moves from a fresh state: x read; Q (bf16) written by the
    state update, read by the score product and again by the state product; a bf16 copy of the state per 256-token
    chunk but the first, written and read; the f32 state written; out written."""
    S, nc = B * h, T // 256
    q = 2.0 * S * T * N
    state_copy = 2.0 * S * N * d
    return q + (q + 2 * q) + 2 * (nc - 1) * state_copy + 4.0 * S * N * d + 4.0 * S * T * d


def bench_prefill(args):
    """BASELINE config 3 (see measure_prefill)."""
    B = 8 if args.batch == 32 else args.batch
    h, N, d, T = args.heads, args.latent, args.embd, args.time
    steps = min(args.steps, 20) if args.steps == 1000 else args.steps
    warmup = min(args.warmup, 3) if args.warmup == 50 else args.warmup
    ms, flop = measure_prefill(B, h, N, d, T, args.density, steps, warmup, args.rotary, args.row_normalize,
                               args.all_scores)
    achieved = flop / (ms * 1e-3) / 1e12
    plain = args.rotary == "rope" and not args.row_normalize
    chunked = plain and not args.all_scores and d == 256 and N % 256 == 0 and T % 256 == 0
    executed = prefill_executed_flop(B, h, N, d, T) if chunked else None
    print(json.dumps({
        "metric": "prefill tokens/sec (chunked dense linear attention) + bf16 MFMA utilisation",
        "value": B * T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"BASELINE config 3: chunked prefill B={B} T={T} h={h} N={N} d={d}, bf16 in / f32 "
                               f"accumulate, {args.density:.0%} active, {args.rotary} positions 0..T, fresh state"
                               + (", row-normalised stateless form (time blocks of 64)" if args.row_normalize else "")
                               + ("" if chunked else ", all-scores form"),
                   "algorithmic_flop_per_step": flop, "executed_flop_per_step": executed},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "frac_is": "algorithmic (all-scores) FLOP of the workload / time / peak: a utilisation figure "
                                "for the workload, not matrix-pipe busy time; executed_frac counts what is issued",
                     "executed_tflops": (executed / (ms * 1e-3) / 1e12) if executed else None,
                     "executed_frac": (executed / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS) if executed else None,
                     "traffic": prefill_traffic_bytes(B, h, N, d, T) if chunked else None,
                     "traffic_source": "buffer sizes of the chunk-recurrent form (x, Q written once and read twice, one "
                                       "bf16 state copy per 256 tokens written and read, rho, out); counters in "
                                       "profiles/prefill_config3_bf16_kernel_trace.md read the same within 1 %",
                     "hbm_gbs": (prefill_traffic_bytes(B, h, N, d, T) / (ms * 1e-3) / 1e9) if chunked else None,
                     "kernel": "whole bdh_prefill_chunked call (k_state_stream + k_chunk_out); algorithmic FLOP "
                               "= B*h*[T(T-1)N + T(T-1)d + 2TNd], the all-scores count of the workload; the "
                               "chunk-recurrent form executes executed_flop_per_step of them and is bound by its "
                               "HBM traffic (hbm_gbs), not by the matrix cores"},
    }))


def bench_copy(args):
    """Plain device-to-device copy of a known size (1 GiB read + 1 GiB write per step): the
    calibration run for the FETCH_SIZE / WRITE_SIZE counters and a streaming reference point."""
    import torch

    dev = torch.device("cuda:0")
    n = 1 << 28  # f32 elements = 1 GiB
    src = torch.empty(n, device=dev).normal_()
    dst = torch.empty_like(src)
    steps = 20 if args.steps == 1000 else args.steps
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        dst.copy_(src)
    stop.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(stop) / steps
    print(json.dumps({"metric": "device copy bandwidth", "value": 2.0 * n * 4 / (ms * 1e-3) / 1e9, "unit": "GB/s",
                      "n_gpus": 1, "steps": steps, "warmup": 3, "ms_per_step": ms, "higher_is_better": True,
                      "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": "plain copy, 1 GiB read + 1 GiB write per step (counter calibration)",
                                 "bytes_read_per_step": n * 4, "bytes_written_per_step": n * 4}}))


def measure_rmw_ceiling(region_bytes=1 << 30, chunk_kib=2, density=0.0975, lists=16, iters=64, workgroups=8192,
                        modes=(0,)):
    """What the decode step's access pattern reaches with the arithmetic taken away (bdh_probe_chunks):
    random chunk_kib-KiB chunks covering `density` of a region, read, scaled by 1 and written back in place,
    a different ready-made chunk list on every launch.  At the defaults this is the traffic of the config-2
    step (2 KiB = both rows of a lane pair, 9.75 % of 1 GiB = the pair-closed rows at 5 % active neurons).
    Returns {mode: (microseconds per launch, GB/s over bytes read + bytes written)}."""
    import torch

    from burn_dragon_amd import ffi

    dev = torch.device("cuda:0")
    ctx = ffi.default_context(0)
    region = torch.zeros(region_bytes // 4, device=dev)
    n_region = region_bytes // (chunk_kib << 10)
    g = torch.Generator(device=dev).manual_seed(11)
    idx = [torch.nonzero(torch.rand(n_region, device=dev, generator=g) < density).flatten().to(torch.int32).contiguous()
           for _ in range(lists)]
    moved = float(np.mean([i.numel() for i in idx])) * (chunk_kib << 10)
    out = {}
    for mode in modes:
        def launch(i):
            ctx.check(ctx.lib.bdh_probe_chunks(ctx.handle, region.data_ptr(), region_bytes, idx[i % lists].data_ptr(),
                                               idx[i % lists].numel(), chunk_kib, mode, workgroups))
        for i in range(lists):
            launch(i)
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(iters):
            launch(i)
        stop.record()
        torch.cuda.synchronize()
        us = start.elapsed_time(stop) / iters * 1e3
        out[mode] = (us, (2.0 if mode == 0 else 1.0) * moved / (us * 1e-6) / 1e9)
    return out, moved


def measure_deferred(B=32, h=4, N=8192, d=256, density=0.05, rho_dtype="f32", capacity=128, steps=1000, warmup=128,
                     ring=None, seed=2):
    """The decode step with deferred updates (bdh_state_step_deferred) on the config-2 workload: every step reads its
    active rows and logs its update; every `capacity` steps the step itself flushes the log into the state, and a
    final bdh_state_flush ends the run -- ALL flushes are inside the timed region.  The ring holds at least
    `capacity` distinct x sets, so the rows a flush rewrites are the union of that many independent steps.
    Algorithmic bytes are those of the eager step (every touched row read once and written once per step)."""
    import torch
    from scipy.stats import norm

    from burn_dragon_amd import ffi
    from burn_dragon_amd.kernel.linear_attention import build_freqs
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import StateLog

    dev = torch.device("cuda:0")
    ctx = ffi.default_context(0)
    lib = ctx.lib
    ring = max(ring or 16, capacity)
    g = torch.Generator(device=dev).manual_seed(seed)
    tdt = torch.float32 if rho_dtype == "f32" else torch.bfloat16
    esz = 4 if rho_dtype == "f32" else 2
    rho = (0.01 * torch.randn((B, h, N, d), device=dev, generator=g)).to(tdt).contiguous()
    mu = float(norm.ppf(density))
    xs = [torch.relu(torch.randn((B, h, N), device=dev, generator=g) + mu).contiguous() for _ in range(ring)]
    vs = [torch.randn((B, d), device=dev, generator=g).contiguous() for _ in range(ring)]
    freqs = build_freqs(N, 65536.0, RotaryEmbedding.ROPE).reshape(-1).to(dev)
    out = torch.empty((B, h, d), device=dev)
    rows = torch.zeros((B, h), device=dev, dtype=torch.int32)
    positions = np.random.default_rng(3).integers(0, 4096, size=steps + warmup)
    log = StateLog(B, h, N, d, tdt, capacity)
    R = []
    for i in range(ring):
        ctx.check(lib.bdh_state_step_deferred(ctx.handle, log.handle, xs[i].data_ptr(), vs[i].data_ptr(), freqs.data_ptr(),
                                              0, None, rho.data_ptr(), out.data_ptr(), None, rows.data_ptr()))
        R.append(int(rows.sum().item()))
    R_mean = float(np.mean(R))
    bytes_per_step = 2.0 * R_mean * d * esz + 4.0 * B * h * N + 4.0 * B * d + 4.0 * B * h * d + 4.0 * N
    fn, hnd, lh = lib.bdh_state_step_deferred, ctx.handle, log.handle
    call_args = [(hnd, lh, xs[i % ring].data_ptr(), vs[i % ring].data_ptr(), freqs.data_ptr(), int(positions[i]), None,
                  rho.data_ptr(), out.data_ptr(), None, None) for i in range(steps + warmup)]
    for i in range(warmup):
        ctx.check(fn(*call_args[i]))
    log.flush(rho)  # the timed region starts on an empty log
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    rc_bad = 0
    t0 = time.perf_counter()
    start.record()
    for i in range(warmup, warmup + steps):
        rc_bad |= fn(*call_args[i])
    rc_bad |= lib.bdh_state_flush(hnd, lh, rho.data_ptr())
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ctx.check(rc_bad)
    gpu_ms = start.elapsed_time(stop)
    ms_per_step = max(gpu_ms, wall * 1e3) / steps
    achieved = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    flushes = (steps + capacity - 1) // capacity
    res = {
        "workload": f"bdh_state_step_deferred on config 2 (rho {rho_dtype} [{B},{h},{N},{d}], {density:.0%} active, {ring} input sets): "
                    f"log capacity {capacity}, {steps} timed steps with all {flushes} flushes inside the timed region",
        "log_capacity": capacity, "log_bytes": log.nbytes, "steps": steps, "flushes_timed": flushes,
        "ms_per_step": ms_per_step, "tokens_per_s": B / (ms_per_step * 1e-3),
        "gpu_event_ms_total": gpu_ms, "wall_ms_total": wall * 1e3,
        "touched_rows_per_step": R_mean, "algorithmic_bytes_per_step": bytes_per_step,
        "achieved_gbs": achieved, "frac": achieved / HBM_PEAK_GBS,
        "kernels": "k_step_deferred + k_deferred_finalize per step, k_state_flush per flush; achieved = the eager step's "
                   "algorithmic bytes / ms_per_step (the slower of the HIP-event and the host clock)",
    }
    log.close()
    del rho, xs, vs
    torch.cuda.empty_cache()
    return res


def bench_deferred(args):
    """The deferred-update decode step alone (the default line carries the same figures as its `deferred` record)."""
    r = measure_deferred(args.batch, args.heads, args.latent, args.embd, args.density, args.rho_dtype, args.log_capacity,
                         args.steps, max(args.warmup, args.log_capacity), args.ring)
    print(json.dumps({
        "metric": "decode tokens/sec at batch B (single-layer state step, deferred updates) + achieved HBM GB/s",
        "value": r["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.rho_dtype, "data": "synthetic", "config": r,
        "roofline": {"bound": "hbm", "achieved": r["achieved_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": r["frac"], "traffic": None, "kernel": r["kernels"], "launch_us": r["ms_per_step"] * 1e3},
    }))


def bench_rmw_probe(args):
    """The bandwidth ceiling of the decode step's access pattern, measured on this box."""
    res, moved = measure_rmw_ceiling(modes=(0, 1, 2), iters=256 if args.steps == 1000 else args.steps)
    us, gbs = res[0]
    print(json.dumps({
        "metric": "in-place read-modify-write bandwidth of random 2 KiB chunks (decode-step access pattern)",
        "value": gbs, "unit": "GB/s", "n_gpus": 1, "steps": 256 if args.steps == 1000 else args.steps, "warmup": 16,
        "ms_per_step": us * 1e-3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "bdh_probe_chunks: random 2 KiB chunks, 9.75 % of a 1 GiB region, ready-made chunk "
                               "lists (16, rotating), 8192 workgroups of 4 waves, one wave per KiB",
                   "bytes_read_per_launch": moved, "bytes_written_per_launch": moved,
                   "read_only_us": res[1][0], "read_only_gbs": res[1][1],
                   "write_only_us": res[2][0], "write_only_gbs": res[2][1]},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                     "traffic": None, "kernel": "k_probe_chunks<0>", "launch_us": us},
    }))


F32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense f32 matrix, published


def bench_alibi(args):
    """Single-layer ALiBi state step at the decode shape: the reference's eager decay (a dense pass
    over rho every token, src/model/bdh.rs:299-301) beside the lazily decayed state of this library.
    `value` is the lazy step; the eager figures ride along in config."""
    import torch
    from scipy.stats import norm

    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import recurrent_attention, recurrent_attention_lazy_alibi

    dev = torch.device("cuda:0")
    B, h, N, d = args.batch, args.heads, args.latent, args.embd
    steps = 200 if args.steps == 1000 else args.steps
    warmup = min(args.warmup, 10)
    g = torch.Generator(device=dev).manual_seed(1)
    mu = float(norm.ppf(args.density))
    ring = min(args.ring, 8)
    xs = [torch.relu(torch.randn((B, h, 1, N), device=dev, generator=g) + mu) for _ in range(ring)]
    vs = [torch.randn((B, 1, d), device=dev, generator=g) for _ in range(ring)]
    rho = 0.01 * torch.randn((B, h, N, d), device=dev, generator=g)
    stamps = torch.zeros((B, h, N), device=dev, dtype=torch.int32)
    fz = torch.zeros(N, device=dev)
    rows = float(sum(int((x != 0).sum()) for x in xs)) / ring
    times = {}
    for name in ("eager", "lazy"):
        n = steps if name == "lazy" else max(steps // 10, 5)

        def step(i):
            if name == "eager":
                recurrent_attention(xs[i % ring], vs[i % ring], rho, fz, i, RotaryEmbedding.ALIBI)
            else:
                recurrent_attention_lazy_alibi(xs[i % ring], vs[i % ring], rho, stamps, i)

        for i in range(warmup):
            step(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(n):
            step(warmup + i)
        e1.record()
        torch.cuda.synchronize()
        times[name] = max(e0.elapsed_time(e1), (time.perf_counter() - t0) * 1e3) / n
    lazy_bytes = 2.0 * rows * d * 4 + 8.0 * rows + 4.0 * B * h * N + 4.0 * B * d + 4.0 * B * h * d
    dense_bytes = 2.0 * B * h * N * d * 4
    ms = times["lazy"]
    achieved = lazy_bytes / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "decode tokens/sec at batch B (single-layer ALiBi state step, lazily decayed state)",
        "value": B / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"ALiBi state step, rho f32 [{B},{h},{N},{d}], {args.density:.0%} active, {ring} input sets",
                   "active_rows_per_step": rows, "algorithmic_bytes_per_step": lazy_bytes,
                   "eager_ms_per_step": times["eager"], "eager_dense_bytes_per_step": dense_bytes,
                   "eager_GBps": dense_bytes / (times["eager"] * 1e-3) / 1e9, "speedup": times["eager"] / ms},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "k_step_alibi_lazy_f32 (+ k_step_finalize)"},
    }))


def bench_parallel(args):
    """kernel::linear_attention::fused_state_aligned (src/kernel/linear_attention.rs:11-115) in f32 at the
    config-3 shape: normalised causal linear attention over all tokens at once on the f32 matrix cores."""
    import torch

    from burn_dragon_amd.kernel import BlockPattern2d
    from burn_dragon_amd.kernel.linear_attention import build_freqs, fused_state_aligned
    from burn_dragon_amd.positional import RotaryEmbedding

    dev = torch.device("cuda:0")
    B = 8 if args.batch == 32 else args.batch
    h, N, d, T = args.heads, args.latent, args.embd, args.time
    steps = 5 if args.steps == 1000 else args.steps
    warmup = min(args.warmup, 1)
    g = torch.Generator(device=dev).manual_seed(3)
    q = torch.empty((B, h, T, N), device=dev)
    for b in range(B):
        q[b] = torch.relu(torch.randn((h, T, N), device=dev, generator=g) - 1.6449)
    v = torch.randn((B, 1, T, d), device=dev, generator=g)
    f = build_freqs(N, 65536.0, RotaryEmbedding.ROPE, device=dev)
    layout = BlockPattern2d.dense(64)
    for _ in range(warmup):
        fused_state_aligned(q, v, f, None, layout, RotaryEmbedding.ROPE)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fused_state_aligned(q, v, f, None, layout, RotaryEmbedding.ROPE)
    e1.record()
    torch.cuda.synchronize()
    ms = max(e0.elapsed_time(e1), (time.perf_counter() - t0) * 1e3) / steps
    flop = float(B * h) * (T * (T - 1.0) * N + T * (T - 1.0) * d)
    achieved = flop / (ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "tokens/sec, fused_state_aligned (normalised causal linear attention, f32)",
        "value": B * T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"fused_state_aligned B={B} h={h} T={T} N={N} dv={d}, RoPE, dense time blocks of 64, "
                               f"row_normalize, 5% active", "algorithmic_flop_per_step": flop},
        # six bf16 matrix instructions per f32 one (three-term operand split): the peak is the dense bf16 rate over six
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS / 6.0, "unit": "TFLOP/s",
                     "frac": achieved / (MFMA_BF16_PEAK_TFLOPS / 6.0), "traffic": None,
                     "frac_of_f32_matrix_peak": achieved / F32_MFMA_PEAK_TFLOPS,
                     "kernel": "whole bdh_fused_state_aligned call (k_rotate_f32, k_fsa_gemm_f32 x2 with split-bf16 "
                               "products, k_fsa_row_abs_sum); "
                               "algorithmic FLOP = B*h*[T(T-1)N + T(T-1)d]"},
    }))


def bench_chunks(args):
    """BDH::recurrent_attention (src/model/bdh.rs:258-307) over --time tokens per call at the config-2 state
    shape, f32: the many-token form (dense products on the f32 matrix cores) with the token loop of the
    sparse step kernels timed beside it on the same inputs."""
    import torch
    from scipy.stats import norm

    from burn_dragon_amd import ffi
    from burn_dragon_amd.kernel.linear_attention import build_freqs
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import recurrent_attention

    dev = torch.device("cuda:0")
    B, h, N, d = args.batch, args.heads, args.latent, args.embd
    T = 256 if args.time == 2048 else args.time
    steps = 10 if args.steps == 1000 else args.steps
    warmup = min(args.warmup, 2)
    g = torch.Generator(device=dev).manual_seed(5)
    mu = float(norm.ppf(args.density))
    x = torch.empty((B, h, T, N), device=dev)
    for b in range(B):
        x[b] = torch.relu(torch.randn((h, T, N), device=dev, generator=g) + mu)
    v = torch.randn((B, T, d), device=dev, generator=g)
    rho = 0.01 * torch.randn((B, h, N, d), device=dev, generator=g)
    f = build_freqs(N, 65536.0, RotaryEmbedding.ROPE, device=dev).reshape(-1)
    ctx = ffi.default_context(0)

    def timed(n):
        for _ in range(warmup):
            recurrent_attention(x, v, rho, f, 0, RotaryEmbedding.ROPE)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(n):
            recurrent_attention(x, v, rho, f, i * T, RotaryEmbedding.ROPE)
        e1.record()
        torch.cuda.synchronize()
        return max(e0.elapsed_time(e1), (time.perf_counter() - t0) * 1e3) / n

    ms = timed(steps)
    ctx.set_option("state_step.dense_chunks", 0)
    try:
        ms_loop = timed(max(1, steps // 5))
    finally:
        ctx.set_option("state_step.dense_chunks", -1)
    S = float(B * h)
    flop = S * (T * (T - 1.0) * N + T * (T - 1.0) * d + 4.0 * T * N * d)
    achieved = flop / (ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "tokens/sec, many-token recurrent state step (f32 dense products)",
        "value": B * T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"recurrent_attention B={B} h={h} T={T} N={N} d={d}, f32 state, RoPE, "
                               f"{args.density:.0%} active, state carried from call to call",
                   "algorithmic_flop_per_step": flop, "token_loop_ms_per_step": ms_loop,
                   "token_loop_tokens_per_s": B * T / (ms_loop * 1e-3)},
        # the products run as six bf16 matrix instructions per f32 one (three-term operand split): the peak that
        # bounds them is the dense bf16 rate over six
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS / 6.0, "unit": "TFLOP/s",
                     "frac": achieved / (MFMA_BF16_PEAK_TFLOPS / 6.0), "traffic": None,
                     "frac_of_f32_matrix_peak": achieved / F32_MFMA_PEAK_TFLOPS,
                     "kernel": "whole call (k_rotate_chunk_f32 + 4 k_fsa_gemm_f32 launches, split-bf16 products); "
                               "algorithmic FLOP = B*h*[T(T-1)N + T(T-1)d + 4TNd]"},
    }))


# (n_layer, n_embd, n_head, mlp_internal_dim_multiplier) of the reference's config/{tiny,small,base,large}.toml
SHIPPED_SIZES = {"tiny": (4, 128, 4, 4), "small": (4, 192, 4, 4), "base": (4, 256, 4, 4), "large": (8, 512, 8, 4)}


def bench_model(args):
    """Full-model greedy decode (BDH::forward_with_state per token, argmax on the device).
    c1 = BASELINE config 1 (V=256, d=256, h=4, N=8192, L=6, B=1, 64-byte prompt, 256 tokens);
    c4 = config 4 shapes (d=512, h=8, N=16384, L=12, B=32) with a SHORT prompt: the state is
    established by --prompt tokens, not by the 3584-token prefill the config names."""
    import torch

    import burn_dragon_amd as bda

    dev = torch.device("cuda:0")
    rho_dtype = bda.ffi.F32 if args.rho_dtype == "f32" else bda.ffi.BF16
    weights_note = "random-init weights (about half the neurons active)"
    if args.model_config == "ckpt":
        # the trained checkpoint the reference ships (tiny_shakespeare: L=4, d=128, h=4, N=128, V=69, ALiBi),
        # a copy of which the tests hold as a data fixture; state kept lazily decayed
        directory = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "golden", "tiny_shakespeare")
        model, tok, _ = bda.BDH.from_checkpoint_dir(directory, dev, rho_dtype=rho_dtype, alibi_lazy=True)
        cfg = model.config
        B = 1 if args.batch == 32 else args.batch
        steps = 256 if args.steps == 1000 else args.steps
        text = ("First Citizen:\nBefore we proceed any further, hear me speak.\n\nAll:\nSpeak, speak.\n" * 8)[:args.prompt]
        prompt = torch.tensor([tok.encode(text)] * B)
        weights_note = "trained tiny_shakespeare checkpoint (ALiBi, lazily decayed state)"
    elif args.model_config in SHIPPED_SIZES:
        # the sizes of the reference's config/*.toml (ALiBi, eagerly decayed f32 state), random-init weights
        L_, d_, h_, mult_ = SHIPPED_SIZES[args.model_config]
        cfg = bda.BDHConfig(n_layer=L_, n_embd=d_, n_head=h_, mlp_internal_dim_multiplier=mult_, vocab_size=256)
        cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ALIBI)
        B = 1 if args.batch == 32 else args.batch
        steps = 256 if args.steps == 1000 else args.steps
        model = bda.BDH(cfg, dev, seed=7, rho_dtype=rho_dtype, alibi_lazy=args.alibi_lazy)
        if args.alibi_lazy:
            weights_note += ", lazily decayed state"
        prompt = torch.randint(0, 256, (B, args.prompt), generator=torch.Generator().manual_seed(1))
    else:
        if args.model_config == "c1":
            cfg = bda.BDHConfig(n_layer=6, n_embd=256, n_head=4, mlp_internal_dim_multiplier=128, vocab_size=256)
            B = 1 if args.batch == 32 else args.batch
            steps = 256 if args.steps == 1000 else args.steps
        else:
            cfg = bda.BDHConfig(n_layer=12, n_embd=512, n_head=8, mlp_internal_dim_multiplier=256, vocab_size=256)
            B = args.batch
            steps = 64 if args.steps == 1000 else args.steps
        cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
        model = bda.BDH(cfg, dev, seed=7, rho_dtype=rho_dtype, defer_updates=args.defer)
        if args.defer:
            weights_note += f", state updates deferred (log of {args.defer} steps; flushes inside the timed region)"
        prompt = torch.randint(0, 256, (B, args.prompt), generator=torch.Generator().manual_seed(1))
    state = model.init_state()
    chunk = args.prefill_chunk or args.prompt
    t0 = time.perf_counter()
    for lo in range(0, prompt.shape[1], chunk):  # bounded activation memory; same result as one call
        _, nxt = model.forward_with_state(prompt[:, lo:lo + chunk], state, want_next=True)
        if (lo // chunk) % 16 == 15:
            torch.cuda.synchronize()
            print(f"prefill {lo + chunk}/{args.prompt} tokens, {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    warm = min(args.warmup, 8)
    for _ in range(warm):
        _, nxt = model.forward_with_state(nxt.reshape(B, 1), state, want_next=True)
    torch.cuda.synchronize()
    graph = model.capture_decode_step(state, nxt) if args.graph else None
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    if graph is not None:
        graph.replay(steps)
    else:
        for _ in range(steps):
            _, nxt = model.forward_with_state(nxt.reshape(B, 1), state, want_next=True)
    model.materialize_state(state)  # a deferred state is flushed inside the timed region
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = max(start.elapsed_time(stop), wall * 1e3) / steps
    h, d, N, L = cfg.n_head, cfg.n_embd, cfg.latent_per_head(), cfg.n_layer
    extra = {}
    if args.model_config == "c1" and not args.no_cpu_baseline:
        extra["cpu_baseline"] = cpu_baseline_model(cfg, B, prompt.numpy())
    print(json.dumps({
        "metric": "decode tokens/sec, full model, greedy", "value": B / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.rho_dtype, "data": "synthetic",
        "config": {"workload": f"full-model greedy decode {args.model_config}: L={L} d={d} h={h} N={N} "
                               f"V={cfg.vocab_size} B={B}, {weights_note}, prompt {prompt.shape[1]} tokens"
                               + (", one HIP graph replay per token" if args.graph else ", eager launches"),
                   "prefill_seconds": prefill_s, "prefill_tokens_per_s": B * prompt.shape[1] / prefill_s,
                   "state_bytes": L * B * h * N * d * (4 if args.rho_dtype == "f32" else 2)},
        **extra,
    }))


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--heads", type=int, default=4)
    ap.add_argument("--latent", type=int, default=8192)
    ap.add_argument("--embd", type=int, default=256)
    ap.add_argument("--density", type=float, default=0.05)
    ap.add_argument("--rho-dtype", choices=["f32", "bf16"], default="f32")
    ap.add_argument("--ring", type=int, default=16, help="number of distinct (x, v) input sets")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--log-capacity", type=int, default=128, help="deferred: steps the update log holds between flushes")
    ap.add_argument("--prefill-chunk", type=int, default=0,
                    help="model workload: feed the prompt in calls of this many tokens (0 = one call)")
    ap.add_argument("--workload", choices=["decode", "deferred", "prefill", "model", "copy", "alibi", "parallel", "chunks", "rmw_probe"], default="decode",
                    help="decode = BASELINE config 2 (the headline metric); prefill = config 3 (bf16 MFMA); "
                         "model = full-model greedy decode (config 1 by default, --model-config c4 for config 4); "
                         "alibi = ALiBi state step, lazily decayed state beside the eager dense decay; "
                         "parallel = fused_state_aligned in f32 at the config-3 shape; chunks = many-token state step "
                         "(f32 dense products) beside the token loop at the config-2 shape; copy = counter calibration; "
                         "rmw_probe = the bandwidth the decode step's access pattern reaches without its arithmetic")
    ap.add_argument("--model-config", choices=["c1", "c4", "ckpt", *SHIPPED_SIZES], default="c1",
                    help="model: config 1, config 4, the trained tiny_shakespeare checkpoint of the test fixtures, or one "
                         "of the sizes the reference ships configurations for (random-init, ALiBi)")
    ap.add_argument("--alibi-lazy", action="store_true", help="model, shipped sizes: keep the ALiBi state lazily decayed")
    ap.add_argument("--prompt", type=int, default=64, help="model: prompt tokens per sequence")
    ap.add_argument("--graph", action="store_true", help="model: replay one captured HIP graph per token")
    ap.add_argument("--defer", type=int, default=0, metavar="K",
                    help="model (c1, c4): decode with deferred state updates, a log of K steps per layer")
    ap.add_argument("--time", type=int, default=2048, help="prefill: tokens per sequence")
    ap.add_argument("--rotary", choices=["rope", "alibi", "pope"], default="rope", help="prefill: positional scheme")
    ap.add_argument("--row-normalize", action="store_true",
                    help="prefill: the row-normalised stateless form of fused_state_aligned on the bf16 matrix cores")
    ap.add_argument("--all-scores", action="store_true", help="prefill: never the chunk-recurrent form")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="library launch-shape option set on the context before the run (repeatable)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path has no multi-GPU part); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from scipy.stats import norm

    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible; the HIP path is the only path", file=sys.stderr)
        sys.exit(1)
    from burn_dragon_amd import ffi
    from burn_dragon_amd.kernel.linear_attention import build_freqs
    from burn_dragon_amd.positional import RotaryEmbedding

    dev = torch.device("cuda:0")
    for item in args.option:
        name, _, value = item.partition("=")
        ffi.default_context(0).set_option(name, int(value))
    if args.workload == "prefill":
        return bench_prefill(args)
    if args.workload == "model":
        return bench_model(args)
    if args.workload == "copy":
        return bench_copy(args)
    if args.workload == "alibi":
        return bench_alibi(args)
    if args.workload == "parallel":
        return bench_parallel(args)
    if args.workload == "chunks":
        return bench_chunks(args)
    if args.workload == "rmw_probe":
        return bench_rmw_probe(args)
    if args.workload == "deferred":
        return bench_deferred(args)
    B, h, N, d = args.batch, args.heads, args.latent, args.embd
    ctx = ffi.default_context(0)
    lib = ctx.lib
    g = torch.Generator(device=dev).manual_seed(2)
    tdt = torch.float32 if args.rho_dtype == "f32" else torch.bfloat16
    esz = 4 if args.rho_dtype == "f32" else 2
    rho = (0.01 * torch.randn((B, h, N, d), device=dev, generator=g)).to(tdt).contiguous()
    mu = float(norm.ppf(args.density))
    xs = [torch.relu(torch.randn((B, h, N), device=dev, generator=g) + mu).contiguous() for _ in range(args.ring)]
    vs = [torch.randn((B, d), device=dev, generator=g).contiguous() for _ in range(args.ring)]
    freqs_host = build_freqs(N, 65536.0, RotaryEmbedding.ROPE).reshape(-1)
    freqs = freqs_host.to(dev)
    out = torch.empty((B, h, d), device=dev)
    rows = torch.zeros((B, h), device=dev, dtype=torch.int32)
    positions = np.random.default_rng(3).integers(0, 4096, size=args.steps + args.warmup)
    rdt = ffi.F32 if args.rho_dtype == "f32" else ffi.BF16

    # touched rows per input set (R of the algorithmic-bytes formula), measured by the kernel itself
    R = []
    scratch = rho.clone()
    for i in range(args.ring):
        ctx.check(lib.bdh_state_step(ctx.handle, B, h, N, d, ffi.ROPE, xs[i].data_ptr(), vs[i].data_ptr(),
                                     freqs.data_ptr(), 0, None, None, scratch.data_ptr(), rdt, out.data_ptr(), None,
                                     rows.data_ptr()))
        R.append(int(rows.sum().item()))
    del scratch
    R_mean = float(np.mean(R))
    bytes_per_step = 2.0 * R_mean * d * esz + 4.0 * B * h * N + 4.0 * B * d + 4.0 * B * h * d + 4.0 * N

    default_workload = (B, h, N, d, args.density, args.rho_dtype) == (32, 4, 8192, 256, 0.05, "f32")
    fn, hnd = lib.bdh_state_step, ctx.handle
    call_args = [(hnd, B, h, N, d, ffi.ROPE, xs[i % args.ring].data_ptr(), vs[i % args.ring].data_ptr(),
                  freqs.data_ptr(), int(positions[i]), None, None, rho.data_ptr(), rdt, out.data_ptr(), None, None)
                 for i in range(args.steps + args.warmup)]
    for i in range(args.warmup):
        ctx.check(fn(*call_args[i]))
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    rc_bad = 0
    t0 = time.perf_counter()
    start.record()  # the context launches on torch's current stream, so these events bracket the kernels
    for i in range(args.warmup, args.warmup + args.steps):
        rc_bad |= fn(*call_args[i])
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ctx.check(rc_bad)
    gpu_ms = start.elapsed_time(stop)
    ms_per_step = max(gpu_ms, wall * 1e3) / args.steps  # the slower of the two clocks
    event_us = gpu_ms / args.steps * 1e3
    achieved = bytes_per_step / (ms_per_step * 1e-3) / 1e9  # on the same clock as ms_per_step and value
    ceiling = None
    if default_workload:  # the same pattern without the arithmetic, measured in this run
        probe, _ = measure_rmw_ceiling(iters=64)
        ceiling = probe[0][1]

    result = {
        "metric": "decode tokens/sec at batch B (single-layer state step) + achieved HBM GB/s",
        "value": B * args.steps / (ms_per_step * args.steps * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.rho_dtype,
        "data": "synthetic",
        "config": {
            "workload": f"BASELINE config 2: single-layer decode state step, rho {args.rho_dtype} [{B},{h},{N},{d}], "
                        f"x=relu(N(mu,1)) {args.density:.0%} active, RoPE position ~U[0,4096), {args.ring} input sets",
            "batch": B, "heads": h, "latent_per_head": N, "n_embd": d, "density": args.density,
            "touched_rows_per_step": R_mean, "algorithmic_bytes_per_step": bytes_per_step,
            "gpu_event_ms_total": gpu_ms, "wall_ms_total": wall * 1e3,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a plain copy of
            # known size; measured for the default workload only, by the profile named in traffic_source
            "traffic": 216.06e6 if default_workload else None,
            "traffic_source": ("profiles/state_step_config2_f32_pmc_traffic.md (a constant copied from that "
                               "summary, not re-measured by this run)") if default_workload else None,
            "kernel": f"k_step_rope_{args.rho_dtype} (+ k_step_finalize); achieved = algorithmic bytes / ms_per_step "
                      "(both kernels of the step, the slower of the HIP-event and the host clock)",
            "launch_us": ms_per_step * 1e3,
            "event_us": event_us,
            # the dominant kernel alone, from the committed rocprofv3 kernel trace of this command
            "kernel_us": 42.3 if default_workload else None,
            "kernel_us_source": ("profiles/state_step_config2_f32_kernel_trace.md (a constant copied from that "
                                 "summary; event_us is this run's own clock for both kernels of the step)")
            if default_workload else None,
            # bdh_probe_chunks in this run: in-place read-modify-write of random 2 KiB chunks (9.75 % of 1 GiB)
            # from ready-made lists: what this access pattern reaches with no arithmetic at all
            "ceiling_measured_gbs": ceiling,
            "frac_of_measured_ceiling": (achieved / ceiling) if ceiling else None,
        },
    }
    if default_workload:
        # the same workload through the deferred-update step (flushes inside its timed region)
        del rho, xs, vs
        torch.cuda.empty_cache()
        # its own step count: at least eight log capacities, so that the flushes -- all of them inside its timed
        # region, the final one included -- are amortised as in a decode loop, whatever --steps says for the line's value
        result["deferred"] = measure_deferred(steps=max(args.steps, 8 * 128), warmup=max(args.warmup, 128))
        # BASELINE config 3 beside the headline: the chunked prefill, bf16 matrix cores (its own roofline)
        p_ms, p_flop = measure_prefill(steps=5, warmup=2)
        torch.cuda.empty_cache()
        q_ms = measure_prefill_queued()
        p_exec = prefill_executed_flop(8, 4, 8192, 256, 2048)
        result["prefill_config3"] = {
            "workload": "BASELINE config 3: bdh_prefill_chunked B=8 T=2048 h=4 N=8192 d=256, bf16 in / f32 accumulate, "
                        "5% active, fresh state, 5 timed calls",
            "ms": p_ms, "tokens_per_s": 8 * 2048 / (p_ms * 1e-3),
            "algorithmic_flop": p_flop, "tflops": p_flop / (p_ms * 1e-3) / 1e12,
            # frac: algorithmic (all-scores) FLOP / time / peak, the utilisation the workload's target is stated in;
            # executed_frac: the FLOP the chunk-recurrent form actually issues / time / peak
            "frac": p_flop / (p_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, "peak_tflops": MFMA_BF16_PEAK_TFLOPS,
            "executed_flop": p_exec, "executed_tflops": p_exec / (p_ms * 1e-3) / 1e12,
            "executed_frac": p_exec / (p_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            # what bounds this form: its HBM traffic (buffer sizes; the counters of the profile read the same within 1 %)
            "hbm_traffic_bytes": prefill_traffic_bytes(8, 4, 8192, 256, 2048),
            "hbm_gbs": prefill_traffic_bytes(8, 4, 8192, 256, 2048) / (p_ms * 1e-3) / 1e9,
            "kernel_us_source": "profiles/prefill_config3_bf16_kernel_trace.md",
            # not the latency of a call: the same 8 sequences as two queues of half-batch calls on two streams
            "queued_two_streams_ms_per_8_sequences": q_ms,
            "queued_two_streams_frac": p_flop / (q_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(B, h, N, d, freqs_host.numpy())
    print(json.dumps(result))


if __name__ == "__main__":
    main()
