#!/usr/bin/env python3
"""Benchmark of the op backend's hot path on one MI355X.

A step is one Llama-7B decoder layer's seven Q4_0 x Q8_0 matrix-vector products at m = 1 (q/k/v/o 4096x4096,
gate/up 11008x4096, down 4096x11008), submitted as ONE mailbox message (seven OP_COMPUTE requests) and executed
back-to-back on the context's stream. Weights of LAYERS distinct layers are resident in HBM and steps rotate
through them (LAYERS x 113.8 MB > the 256 MB memory-side cache), so every step streams its weights from HBM.
`value` is algorithmic bytes per step / time per step (weights once, Q8_0 activations once, fp32 outputs once).

The same run also measures, and reports inside the JSON line:
  roofline      the headline shape alone (down-proj GEMV, n = 4096, k = 11008): bytes per launch / average launch
                duration from HIP events on the launching stream, against 8 TB/s
  prefill_gemm  m = 512 Q4_0 GEMM, both shapes of config 2, in int8 Tera-ops/s (2 m n k per launch)
  small_batch   the same layer at m = 8
  q8_0_block    the Qwen2-1.5B-like Q8_0 block of config 4 at m = 1
  cpu_baseline  the scalar C oracle (a port of the same arithmetic) on the host cores, same layer, m = 1
  peaks         MFMA-only loops and a plain copy kernel measured on this device
Every GPU result used for timing is first checked against the oracle on a sample of rows.

usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "htp-ops-lib_amd"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))

import numpy as np  # noqa: E402

HBM_PEAK_GBPS = 8000.0
INT8_PEAK_TOPS = 5000.0
LAYERS = 8
Q4, Q8 = 2, 8


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (every box of this pool has one); --gpus %d is not "
                 "supported. The path shards by output rows (see DESIGN.md) but no multi-GPU code is built." % args.gpus)

    from pyhtpops import api, workloads as wl
    if not os.path.exists(api.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    import oracle_py
    orc = oracle_py.Oracle()
    ctx = api.Context(device=0)

    # ------------------------------------------------------------------ data (outside every timed region)
    t_setup = time.time()
    rng = wl.rng_for(1, 0)
    shapes = wl.LLAMA7B_LAYER
    uniq = {}  # (n, k) -> host weights (one random matrix per shape; layers hold independent device copies)
    for _, n, k in shapes:
        if (n, k) not in uniq:
            uniq[(n, k)] = wl.make_q4_0_weights(rng, n, k)
    acts, act_q, h_act = {}, {}, {}
    for m in (1, 8):
        for k in (4096, 11008):
            x = wl.make_activations(rng, m, k)
            acts[(m, k)] = x
            act_q[(m, k)] = ctx.run_quantize_q8_0(x)                       # quantized on the GPU ...
            assert np.array_equal(act_q[(m, k)], orc.quantize_q8_0(x)), "Q8_0 quantizer is not bit-exact"  # ... bit-exact
            h_act[(m, k)] = ctx.upload(act_q[(m, k)])
    layers = []
    for _ in range(LAYERS):
        layers.append([ctx.upload(uniq[(n, k)]) for _, n, k in shapes])
    h_out = {m: [ctx.alloc(m * n * 4) for _, n, _ in shapes] for m in (1, 8)}
    log("setup: %d layers x %.1f MB of Q4_0 weights resident (%.1f s)" % (
        LAYERS, sum(uniq[(n, k)].nbytes for _, n, k in shapes) / 1e6, time.time() - t_setup))

    def layer_message(layer, m):
        reqs = []
        for i, (_, n, k) in enumerate(shapes):
            body = api.op_compute_request(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0,
                                          api.mat_mul_params((h_out[m][i], 0), (h_act[(m, k)], 0), (layers[layer][i], 0), m, k, n))
            reqs.append((api.REQUEST_TYPE_OP_COMPUTE, body))
        return api.build_message(reqs)

    def check_states(msg):
        st = api.message_request_states(msg)
        if any(s != 0 for s in st):
            raise RuntimeError("a request failed: %r (%s)" % (st, ctx.last_error()))

    # ------------------------------------------------------------------ parity before timing
    def check_layer(m):
        msg = layer_message(0, m)
        assert ctx.process_message(msg) == 0
        check_states(msg)
        worst = 0.0
        for i, (_, n, k) in enumerate(shapes):
            got = ctx.read(h_out[m][i], np.float32, m * n).reshape(m, n)
            rows = np.unique(np.linspace(0, n - 1, 96).astype(int))
            want, mag = orc.mat_mul_q8_0_act_f64(act_q[(m, k)], uniq[(n, k)][rows], m, k, len(rows), Q4)
            err = np.abs(got[:, rows] - want) / mag
            worst = max(worst, float(err.max()))
            assert np.all(err <= 1e-5), "matmul %d outside 1e-5 relative: %g" % (i, err.max())
        return worst

    log("parity m=1: worst |err|/sum|terms| = %.2e; m=8: %.2e" % (check_layer(1), check_layer(8)))

    layer_bytes = {m: sum(wl.matmul_algorithmic_bytes(m, k, n, Q4) for _, n, k in shapes) for m in (1, 8)}

    def time_layers(m, steps, warmup):
        msgs = [layer_message(l, m) for l in range(LAYERS)]
        # steps are enqueued without waiting in between (several messages in flight on the in-order stream);
        # completion of every message is published after the timed region
        for s in range(warmup):
            ctx.enqueue_message(msgs[s % LAYERS])
        ctx.synchronize()
        t0 = time.perf_counter()
        ctx.timer_start()
        for s in range(steps):
            ctx.enqueue_message(msgs[s % LAYERS])
        ev_ms = ctx.timer_stop_ms()
        ctx.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        for msg in msgs:
            ctx.finish_message(msg)
            check_states(msg)
        return ev_ms / steps, wall_ms / steps

    ms_step, wall_step = time_layers(1, args.steps, args.warmup)
    value = layer_bytes[1] / (ms_step * 1e-3) / 1e9
    log("layer m=1: %.2f us/step (events) %.2f us/step (wall)  %.0f GB/s" % (ms_step * 1e3, wall_step * 1e3, value))

    # ------------------------------------------------------------------ headline shape alone (roofline)
    def time_single(n, k, m, wt, handles, h_a, h_o, reps, op):
        reqs = [(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((h_o, 0), (h_a, 0), (h, 0), m, k, n)))
                for h in handles]
        msg = api.build_message(reqs)
        for _ in range(3):
            ctx.process_message(msg)
        ctx.timer_start()
        for _ in range(reps):
            ctx.process_message(msg)
        ms = ctx.timer_stop_ms()
        check_states(msg)
        return ms * 1e3 / (reps * len(handles))  # us per launch

    down = [layers[l][6] for l in range(LAYERS)]
    extra_down = [ctx.upload(uniq[(4096, 11008)]) for _ in range(8)]  # 16 x 25.4 MB = 406 MB of distinct buffers
    us_down = time_single(4096, 11008, 1, Q4, down + extra_down, h_act[(1, 11008)], h_out[1][6], 30, api.HTP_OPS_MAT_MUL_Q4_0_Q8_0)
    us_down_hot = time_single(4096, 11008, 1, Q4, down[:1] * 16, h_act[(1, 11008)], h_out[1][6], 30, api.HTP_OPS_MAT_MUL_Q4_0_Q8_0)
    bytes_down = wl.matmul_algorithmic_bytes(1, 11008, 4096, Q4)
    gbps_down = bytes_down / us_down / 1e3
    log("down-proj GEMV 4096x11008: %.2f us cold (%.0f GB/s, %.1f%% of 8 TB/s); %.2f us cache-resident" % (
        us_down, gbps_down, gbps_down / 80, us_down_hot))
    for h in extra_down:
        ctx.release(h)

    # ------------------------------------------------------------------ m = 8
    ms_step8, _ = time_layers(8, max(20, args.steps // 4), 5)
    log("layer m=8: %.2f us/step  %.0f GB/s" % (ms_step8 * 1e3, layer_bytes[8] / ms_step8 / 1e6))

    # ------------------------------------------------------------------ prefill GEMM (config 2)
    prefill = []
    rng2 = wl.rng_for(2, 0)
    for (n, k) in ((11008, 4096), (4096, 11008)):
        m = 512
        x = wl.make_activations(rng2, m, k)
        aq = ctx.run_quantize_q8_0(x)
        ha, ho = ctx.upload(aq), ctx.alloc(m * n * 4)
        hw = layers[0][4] if (n, k) == (11008, 4096) else layers[0][6]
        us = time_single(n, k, m, Q4, [hw], ha, ho, 10, api.HTP_OPS_MAT_MUL_Q4_0_Q8_0)
        got = ctx.read(ho, np.float32, m * n).reshape(m, n)
        rows_m = [0, 257, 511]
        cols = np.unique(np.linspace(0, n - 1, 64).astype(int))
        want, mag = orc.mat_mul_q8_0_act_f64(aq[rows_m], uniq[(n, k)][cols], len(rows_m), k, len(cols), Q4)
        assert np.all(np.abs(got[np.ix_(rows_m, cols)] - want) <= 1e-5 * mag), "prefill GEMM outside 1e-5 relative"
        tops = 2.0 * m * n * k / us / 1e6
        prefill.append({"m": m, "n": n, "k": k, "us": round(us, 2), "tera_ops": round(tops, 1),
                        "frac_of_int8_nominal": round(tops / INT8_PEAK_TOPS, 4),
                        "algorithmic_bytes": wl.matmul_algorithmic_bytes(m, k, n, Q4)})
        log("prefill GEMM m=512 n=%d k=%d: %.1f us  %.1f Tops (%.1f%% of 5 Pop/s)" % (n, k, us, tops, tops / 50))
        ctx.release(ha), ctx.release(ho)

    # ------------------------------------------------------------------ Q8_0 block (config 4), m = 1
    rng4 = wl.rng_for(4, 0)
    q8_bytes, q8_us = 0, 0.0
    for name, n, k in wl.QWEN2_1P5B_LAYER:
        if name in ("k", "o", "up"):
            continue  # same shapes as q, v, gate: measured once, counted twice below
        w8 = wl.make_q8_0_weights(rng4, n, k)
        copies = [ctx.upload(w8) for _ in range(max(2, int(300e6 // w8.nbytes)))]
        aq = ctx.run_quantize_q8_0(wl.make_activations(rng4, 1, k))
        ha, ho = ctx.upload(aq), ctx.alloc(n * 4)
        us = time_single(n, k, 1, Q8, copies, ha, ho, 5, api.HTP_OPS_MAT_MUL_Q8_0_Q8_0)
        got = ctx.read(ho, np.float32, n)
        want, mag = orc.mat_mul_q8_0_act_f64(aq, w8[:64], 1, k, 64, Q8)
        assert np.all(np.abs(got[:64] - want[0]) <= 1e-5 * mag[0])
        mult = 2 if name in ("q", "v", "gate") else 1
        q8_bytes += mult * wl.matmul_algorithmic_bytes(1, k, n, Q8)
        q8_us += mult * us
        for h in copies + [ha, ho]:
            ctx.release(h)
    log("Q8_0 block m=1: %.1f us for 7 GEMVs, %.0f GB/s" % (q8_us, q8_bytes / q8_us / 1e3))

    # ------------------------------------------------------------------ device ceilings
    peaks = {
        "mfma_i8_32x32x32_tera_ops": round(ctx.measure_mfma_peak(0, 20000), 1),
        "mfma_i8_16x16x64_tera_ops": round(ctx.measure_mfma_peak(1, 20000), 1),
        "mfma_f16_32x32x16_tera_flops": round(ctx.measure_mfma_peak(2, 20000), 1),
        "copy_kernel_GBps_read_plus_write_1GiB": round(ctx.measure_copy_bandwidth(1 << 30, 10), 0),
    }
    log("device ceilings:", peaks)

    # ------------------------------------------------------------------ CPU baseline: the oracle on the host cores
    cpu = None
    if not args.skip_cpu:
        try:
            native = oracle_py.Oracle(oracle_py.build(native=True))
        except Exception as e:  # no compiler on this machine: time the portable build
            log("native oracle build failed (%s); timing the portable build" % e)
            native = orc
        cores = min(os.cpu_count() or 1, 16)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 10.0:
            for _, n, k in shapes:
                native.mat_mul_q8_0_act(act_q[(1, k)], uniq[(n, k)], 1, k, n, Q4, n_threads=cores)
            reps += 1
        t_mt = (time.perf_counter() - t0) / reps
        t0 = time.perf_counter()
        for _, n, k in shapes:
            native.mat_mul_q8_0_act(act_q[(1, k)], uniq[(n, k)], 1, k, n, Q4, n_threads=1)
        t_1 = time.perf_counter() - t0
        cpu = {"value": round(layer_bytes[1] / t_mt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": "the same 7-GEMV layer at m=1 with the scalar C oracle (gcc -O3 -march=native, pthreads over output "
                         "rows), %d passes in ~10 s" % reps,
               "us_per_step": round(t_mt * 1e6, 1),
               "single_thread_GBps": round(layer_bytes[1] / t_1 / 1e9, 3)}
        log("CPU baseline: %.2f GB/s on %d threads (%.0f us/layer); 1 thread %.3f GB/s" % (
            cpu["value"], cores, t_mt * 1e6, cpu["single_thread_GBps"]))

    result = {
        "metric": "Q4_0 GEMV HBM GB/s (% peak) + M=512 prefill int8 MFMA TOPS, 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "configs[1]: Llama-7B decode layer, 7 Q4_0xQ8_0 GEMVs at m=1 submitted as one message, "
                               "%d layers of distinct weights rotated (cold HBM reads)" % LAYERS,
                   "algorithmic_bytes_per_step": layer_bytes[1], "pct_of_hbm_peak": round(value / HBM_PEAK_GBPS * 100, 2),
                   "wall_ms_per_step": round(wall_step, 6)},
        "roofline": {"bound": "hbm", "achieved": round(gbps_down, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps_down / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "gemv_shared_act_kernel<Q4_0> n=4096 k=11008 m=1", "bytes_per_launch": bytes_down,
                     "us_per_launch": round(us_down, 3), "us_per_launch_cache_resident": round(us_down_hot, 3)},
        "cpu_baseline": cpu,
        "prefill_gemm": prefill,
        "small_batch": {"m": 8, "us_per_step": round(ms_step8 * 1e3, 2),
                        "GBps": round(layer_bytes[8] / ms_step8 / 1e6, 1)},
        "q8_0_block": {"m": 1, "us_7_gemvs": round(q8_us, 2), "GBps": round(q8_bytes / q8_us / 1e3, 1)},
        "peaks": peaks,
    }
    ctx.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
