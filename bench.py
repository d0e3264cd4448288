#!/usr/bin/env python3
"""Benchmark of the quantized-matmul path on one MI355X.

A step is one decode-step matmul sweep of a Qwen2.5-0.5B-shaped model at batch 1 with
per-row int8 weights: 24 layers x {q, k, v, o, gate, up, down} + lm_head = 169 calls of
pytorch_linear, enqueued in order on one stream (weights, activations and outputs are
resident in HBM before the timed region starts).  `value` is the algorithmic bytes of
the sweep (weights + scales, 494 873 344 B) divided by the time per step.

Also reported on the same JSON line:
  roofline     - the lm_head int8 GEMV kernel alone (W[151936x896], 136 744 192 algorithmic
                 bytes per launch), timed with HIP events on the launch stream over a run of
                 launches that rotates through enough weight copies to exceed the 256 MB
                 last-level cache, so every launch streams from HBM;
  cpu_baseline - the CPU oracle (a C restatement of the reference kernels, OpenMP over rows)
                 on a bounded sample of the same sweep, on the host cores of this box;
  detail       - per-config figures (int8 / Q4 / fp16 GEMV shapes).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

H, INTER, KV, VOCAB, LAYERS = 896, 4864, 128, 151936, 24
LAYER_SHAPES = [("q", H, H), ("k", KV, H), ("v", KV, H), ("o", H, H),
                ("gate", INTER, H), ("up", INTER, H), ("down", H, INTER)]
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the lm_head int8 GEMV kernel, from rocprofv3 FETCH_SIZE and WRITE_SIZE
# (separate counter runs of this script, scaled by what the same counters read for a
# device-to-device copy of known size; profiles/gemv_int8_lm_head_hbm_traffic.txt).
LM_HEAD_I8_TRAFFIC_BYTES = 142203900


def algo_bytes_i8(N, K):
    return N * K + 2 * N + 2 * K + 2 * N          # weights + scales + x + y


def algo_bytes_q4(N, K):
    return N * K // 2 + 2 * N * (K // 32) + 2 * K + 2 * N


def algo_bytes_f16(N, K):
    return 2 * N * K + 2 * K + 2 * N


def time_region(mil, queue, fn, reps, samples=1):
    """ms per call of fn: `samples` regions of `reps` calls each, bracketed by HIP events on the
    launch stream; the median region (samples = 1: that one region)."""
    e0, e1 = mil.Event(), mil.Event()
    got = []
    for _ in range(samples):
        queue.finish()
        e0.record(queue)
        for _ in range(reps):
            fn()
        e1.record(queue)
        e1.synchronize()
        queue.finish()
        got.append(e0.elapsed_ms(e1) / reps)
    got.sort()
    return got[len(got) // 2]


def host_cpu():
    """(model string, cores this process may run on, cores online) of the host."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = os.cpu_count()
    return model, allowed, os.cpu_count()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-detail", action="store_true", help="skip the per-config detail runs")
    ap.add_argument("--no-graph", action="store_true",
                    help="time stream launches only (rocprofv3's kernel trace crashes in hipGraphLaunch)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        return 2

    mil = importlib.import_module("adreno-llms_amd")
    assert mil.lib().mi_init(0) == 1, "bench: no gfx950 device"
    queue = mil.Queue()
    t_setup = time.time()

    # ---- synthetic model: W ~ N(0, 0.02) fp16, quantised per row to int8 ------------------
    def make_i8(seed, N, K):
        w = mil.synth_normal_f16(seed, 0.02, (N, K))
        q, s = mil.quantize_int8(w)
        qb, sb = mil.Buffer.from_host(q), mil.Buffer.from_host(s)
        assert mil.nnopt_register_int8_weight(qb, sb, N, K)
        return qb, sb, (q, s)

    # Buffers follow the data flow of a decode step, so that the launches depend on each
    # other as they do in the model (the attention and SwiGLU kernels that sit between the
    # projections are not part of this path and are left out): hidden -> q,k,v ; q -> o ;
    # o -> gate,up ; gate -> down ; down is the next layer's hidden ; last hidden -> lm_head.
    keep, calls, call_family = [], [], []
    x_h = mil.Buffer.from_host(mil.synth_normal_f16(1, 1.0, (H,)))
    x_i = mil.Buffer.from_host(mil.synth_normal_f16(2, 1.0, (INTER,)))
    outs = {n: mil.Buffer(N * 2) for n, N, _ in LAYER_SHAPES}
    hidden = [mil.Buffer.from_host(mil.synth_normal_f16(3, 1.0, (H,))), mil.Buffer(H * 2)]
    logits = mil.Buffer(VOCAB * 2)
    sweep_bytes = 0
    host_layer0 = {}
    layer_w = [dict() for _ in range(LAYERS)]
    for layer in range(LAYERS):
        for j, (name, N, K) in enumerate(LAYER_SHAPES):
            qb, sb, host = make_i8(1000 + layer * 16 + j, N, K)
            keep += [qb, sb]
            layer_w[layer][name] = qb
            if layer == 0:
                host_layer0[name] = host
            cur, nxt = hidden[layer % 2], hidden[(layer + 1) % 2]
            src = {"q": cur, "k": cur, "v": cur, "o": outs["q"], "gate": outs["o"], "up": outs["o"],
                   "down": outs["gate"]}[name]
            calls.append((1, N, K, src, qb, nxt if name == "down" else outs[name]))
            call_family.append({"q": "qkv", "k": "qkv", "v": "qkv", "o": "o", "gate": "gate_up", "up": "gate_up",
                                "down": "down"}[name])
            sweep_bytes += N * K + 2 * N
    lm_q, lm_s, lm_host = make_i8(7, VOCAB, H)
    calls.append((1, VOCAB, H, hidden[LAYERS % 2], lm_q, logits))
    call_family.append("lm_head")
    sweep_bytes += VOCAB * H + 2 * VOCAB
    assert sweep_bytes == 494873344, sweep_bytes
    call_arr = mil.make_calls(calls)
    setup_s = time.time() - t_setup

    # ---- the sweep: stream launches and graph replay --------------------------------------
    def sweep_stream():
        n = mil.linear_batch(queue, call_arr)
        assert n == len(call_arr)

    for _ in range(args.warmup):
        sweep_stream()
    ms_stream = time_region(mil, queue, sweep_stream, args.steps)

    ms_graph = float("inf")
    if not args.no_graph:
        with mil.Graph(queue) as graph:
            sweep_stream()
        for _ in range(args.warmup):
            graph.launch()
        ms_graph = time_region(mil, queue, graph.launch, args.steps)

    launch_mode = "hip_graph" if ms_graph < ms_stream else "stream"
    ms_step = min(ms_graph, ms_stream)
    # the same step as the median of ten shorter regions (the headline is the mean over all K steps)
    per = max(1, args.steps // 10)
    ms_step_median = time_region(mil, queue, sweep_stream if launch_mode == "stream" else graph.launch, per, 10)
    value = sweep_bytes / (ms_step * 1e-3) / 1e9

    # ---- roofline of the dominant kernel: lm_head int8 GEMV, cold ---------------------------
    copies = [(lm_q, lm_s)]
    for c in range(2):                       # 3 x 136 MB > 256 MB of last-level cache
        qb, sb = mil.Buffer(VOCAB * H), mil.Buffer(VOCAB * 2)
        mil.lib().mi_memcpy_d2d(qb.ptr, lm_q.ptr, VOCAB * H, queue.handle)
        mil.lib().mi_memcpy_d2d(sb.ptr, lm_s.ptr, VOCAB * 2, queue.handle)
        assert mil.nnopt_register_int8_weight(qb, sb, VOCAB, H)
        copies.append((qb, sb))
    queue.finish()
    lm_calls = mil.make_calls([(1, VOCAB, H, x_h, copies[i % 3][0], logits) for i in range(30)])
    for _ in range(2):
        mil.linear_batch(queue, lm_calls)
    ms_lm = time_region(mil, queue, lambda: mil.linear_batch(queue, lm_calls), 2, 9) / 30
    lm_bytes = algo_bytes_i8(VOCAB, H)
    achieved = lm_bytes / (ms_lm * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": "gemv int8 K=896 (lm_head, N=151936)", "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": LM_HEAD_I8_TRAFFIC_BYTES,
                "traffic_source": "constant from profiles/gemv_int8_lm_head_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE, "
                                  "WRITE_SIZE of this kernel, scaled by a copy of known size); not measured by this run",
                "us_per_launch": round(ms_lm * 1e3, 2), "bytes_per_launch": lm_bytes,
                "timing": "median of 9 regions of 60 launches, HIP events on the launch stream, weights rotate through "
                          "3 copies (408 MB) so every launch streams from HBM"}

    # ---- per-config detail -------------------------------------------------------------------
    detail = {"decode_step_us_stream": round(ms_stream * 1e3, 1), "decode_step_us_graph": None if args.no_graph else round(ms_graph * 1e3, 1),
              "decode_step_us_median_of_10_regions": round(ms_step_median * 1e3, 1), "setup_s": round(setup_s, 1)}

    # ---- the launches the step's time goes to: each family of launches timed by leaving it out ----
    # (a launch inside a chain of dependent launches cannot be bracketed by events without changing
    # the chain; the sweep without one family, weights as cold as in the full sweep, can)
    if True:                            # also without --detail: roofline.by_time comes from here
        fam_rows = {"qkv": H + 2 * KV, "o": H, "gate_up": 2 * INTER, "down": H, "lm_head": VOCAB}
        fam_k = {"qkv": H, "o": H, "gate_up": H, "down": INTER, "lm_head": H}
        by_time = []
        for fam in ("gate_up", "down", "qkv", "o", "lm_head"):
            sub = mil.make_calls([c for c, f in zip(calls, call_family) if f != fam])
            run = lambda: mil.linear_batch(queue, sub)
            if not args.no_graph:
                with mil.Graph(queue) as gsub:
                    mil.linear_batch(queue, sub)
                run = gsub.launch
            for _ in range(5):
                run()
            ms_without = time_region(mil, queue, run, per, 10)
            n_launch = 1 if fam == "lm_head" else LAYERS
            us = max(ms_step_median - ms_without, 1e-6) * 1e3 / n_launch
            nbytes = fam_rows[fam] * fam_k[fam] + 4 * fam_rows[fam] + 2 * fam_k[fam]
            by_time.append({"kernel": f"gemv int8 {fam} ({fam_rows[fam]} rows x {fam_k[fam]}), one launch",
                            "launches_per_step": n_launch, "bytes_per_launch": nbytes, "us_per_launch": round(us, 2),
                            "achieved": round(nbytes / us / 1e3, 1), "unit": "GB/s", "peak": HBM_PEAK_GBS,
                            "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                            "share_of_step": round(us * n_launch / (ms_step_median * 1e3), 3)})
        how = ("time of the sweep minus time of the sweep without that family of launches (median of 10 regions each), "
               "per launch; bound hbm; the launches are latency-bound, see frac")
        detail["roofline_by_time"] = {"how": how, "kernels": by_time}
        # the launch the step spends most of its time in, beside the launch that moves most of its bytes
        top = max(by_time, key=lambda k: k["share_of_step"])
        roofline["by_time"] = dict(top, bound="hbm", how=how)
        roofline["step"] = {"achieved": round(value, 1), "unit": "GB/s", "peak": HBM_PEAK_GBS,
                            "frac": round(value / HBM_PEAK_GBS, 4),
                            "note": "the whole sweep (this line's value): 97 dependent launches, most of them bound by "
                                    "the launch floor, not by bytes; `kernel` above is the one launch large enough to "
                                    "show a bandwidth and takes share_of_step " +
                                    str(next(k["share_of_step"] for k in by_time if "lm_head" in k["kernel"]))}

    # ---- what a pure reader gets: the practical ceiling beside the 8 TB/s peak ------------------
    # (the reference's gemv_stream_buf probe, QW/kernels/gemv_m1.cl:105-131); the three lm_head copies
    # are contiguous enough for this purpose: each launch reads one copy, rotating
    def read_probe(nbytes):
        fn = lambda: [mil.lib().mi_stream_read_probe(queue.handle, copies[i % 3][0].ptr, nbytes, None) for i in range(30)]
        fn()
        ms = time_region(mil, queue, fn, 2, 9) / 30
        return {"bytes": nbytes, "us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                "frac_hbm": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    detail["read_probe_int8_lm_head_bytes"] = read_probe(VOCAB * H)
    detail["read_probe_q4_lm_head_bytes"] = read_probe(algo_bytes_q4(VOCAB, H) // 16 * 16)
    roofline["frac_of_read_probe"] = round(detail["read_probe_int8_lm_head_bytes"]["us"] / roofline["us_per_launch"], 4)
    if not args.no_detail:
        def cold_gemv(kind, N, K, reps_pool):
            """us per launch over a pool of distinct weights larger than the last-level cache."""
            w = mil.synth_normal_f16(99, 0.02, (N, K))
            if kind == "i8":
                a, b = mil.quantize_int8(w)
                nbytes = algo_bytes_i8(N, K)
            elif kind == "q4":
                a, b = mil.quantize_q4(w)
                nbytes = algo_bytes_q4(N, K)
            else:
                a, b = w, None
                nbytes = algo_bytes_f16(N, K)
            pool = []
            npool = max(3, min(reps_pool, int(600e6 // a.nbytes) + 1))
            for _ in range(npool):
                wb = mil.Buffer.from_host(a)
                sb = mil.Buffer.from_host(b) if b is not None else None
                if kind == "i8":
                    assert mil.nnopt_register_int8_weight(wb, sb, N, K)
                elif kind == "q4":
                    assert mil.nnopt_register_q4_weight(wb, sb, N, K)
                pool.append((wb, sb))
            xb = x_i if K == INTER else x_h
            yb = mil.Buffer(N * 2)
            arr = mil.make_calls([(1, N, K, xb, pool[i % npool][0], yb) for i in range(max(npool, 32))])
            mil.linear_batch(queue, arr)
            ms = time_region(mil, queue, lambda: mil.linear_batch(queue, arr), 1, 7) / len(arr)
            if not args.no_graph:
                with mil.Graph(queue) as g:
                    mil.linear_batch(queue, arr)
                g.launch()
                ms = min(ms, time_region(mil, queue, g.launch, 1, 7) / len(arr))
            # warm: the same weights every launch (they stay in the last-level cache)
            # (timed like the cold figure: the faster of stream launches and graph replay)
            warm = mil.make_calls([(1, N, K, xb, pool[0][0], yb)] * 32)
            mil.linear_batch(queue, warm)
            ms_warm = time_region(mil, queue, lambda: mil.linear_batch(queue, warm), 1, 7) / 32
            if not args.no_graph:
                with mil.Graph(queue) as gw:
                    mil.linear_batch(queue, warm)
                gw.launch()
                ms_warm = min(ms_warm, time_region(mil, queue, gw.launch, 1, 7) / 32)
            for wb, _ in pool:
                mil.nnopt_unregister_weight(wb)
            return {"us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "bytes": nbytes,
                    "us_warm": round(ms_warm * 1e3, 2)}

        detail["c1_fp16_gemv_1536x576"] = cold_gemv("f16", 1536, 576, 340)
        detail["c2_int8_gemv_4864x896"] = cold_gemv("i8", INTER, H, 140)
        detail["c2_int8_gemv_896x4864"] = cold_gemv("i8", H, INTER, 140)
        detail["c3_q4_gemv_151936x896"] = cold_gemv("q4", VOCAB, H, 4)
        detail["c3_q4_gemv_151936x896"]["gemv_mode"] = 1      # the throughput kernel: within 1e-3 / cosine 0.9999 of the oracle
        mil.lib().mi_set_gemv_mode(0)
        try:
            detail["c3_q4_gemv_151936x896_exact_order"] = cold_gemv("q4", VOCAB, H, 4)
            detail["c3_q4_gemv_151936x896_exact_order"]["gemv_mode"] = 0   # bit-identical to the oracle
        finally:
            mil.lib().mi_set_gemv_mode(1)
        for key in ("c3_q4_gemv_151936x896", "c3_q4_gemv_151936x896_exact_order"):
            detail[key]["frac_of_read_probe"] = round(detail["read_probe_q4_lm_head_bytes"]["us"] / detail[key]["us"], 4)
        detail["c3_int8_gemv_151936x896"] = {"us": roofline["us_per_launch"], "GBps": roofline["achieved"],
                                             "frac_hbm": roofline["frac"], "bytes": lm_bytes}
        # the same streaming structure on fp16 weights (no config asks for it at this size): what the launch
        # reaches when the arithmetic per byte is a quarter of int8's in the reference's order
        detail["fp16_gemv_151936x896"] = cold_gemv("f16", VOCAB, H, 3)
        # the fused epilogues at the boundary (int8, warm): residual add, gate/up + SwiGLU, w3 + silu_mul
        def fused_us(fn, n=32):
            fn()
            return round(time_region(mil, queue, lambda: [fn() for _ in range(n)], 1, 7) / n * 1e3, 2)
        wq = {}
        for name, (N, K) in (("down", (H, INTER)), ("gate", (INTER, H)), ("up", (INTER, H))):
            a_, b_ = mil.quantize_int8(mil.synth_normal_f16(300 + len(wq), 0.02, (N, K)))
            wq[name] = (mil.Buffer.from_host(a_), mil.Buffer.from_host(b_))
            assert mil.nnopt_register_int8_weight(wq[name][0], wq[name][1], N, K)
        res_b, act_b = mil.Buffer(H * 2), mil.Buffer(INTER * 2)
        detail["fused_int8_down_plus_residual_896x4864"] = {
            "us_warm": fused_us(lambda: mil.pytorch_linear_add(queue, 1, H, INTER, x_i, wq["down"][0], res_b))}
        detail["fused_int8_gate_up_silu_4864x896"] = {
            "us_warm": fused_us(lambda: mil.fused_gate_up_silu_m1(queue, INTER, H, x_h, wq["gate"][0], wq["up"][0], act_b))}
        detail["fused_int8_w3_silu_gate_4864x896"] = {
            "us_warm": fused_us(lambda: mil.pytorch_linear_silu_gate_fused(queue, INTER, H, x_h, wq["up"][0], act_b))}
        for wb_, _ in wq.values():
            mil.nnopt_unregister_weight(wb_)

        # the greedy step's lm_head: GEMV + argmax, token left in device memory
        token = mil.Buffer(4)

        def lm_head_argmax():
            for i in range(30):
                assert mil.pytorch_linear_argmax(queue, VOCAB, H, x_h, copies[i % 3][0], logits, token)

        lm_head_argmax()
        detail["c4_lm_head_int8_plus_argmax"] = {"us": round(time_region(mil, queue, lm_head_argmax, 1, 7) / 30 * 1e3, 2)}

    # ---- config 4, whole step: every kernel of a greedy decode step on the device -----------
    if not args.no_detail and not args.no_graph:
        one = np.float16(1.0)
        vec = lambda seed, n, base=0.0: mil.Buffer.from_host(np.float16(base) + mil.synth_normal_f16(seed, 0.02, (n,)))
        QD, KVD = 14 * 64, 2 * 64
        dec_w = dict(embed=mil.Buffer.from_host(mil.synth_normal_f16(5000, 0.02, (VOCAB, H))),
                     final_norm=vec(5001, H, 1.0), lm_head=lm_q,
                     in_norm=[vec(5100 + l, H, 1.0) for l in range(LAYERS)],
                     post_norm=[vec(5200 + l, H, 1.0) for l in range(LAYERS)],
                     bq=[vec(5300 + l, QD) for l in range(LAYERS)], bk=[vec(5400 + l, KVD) for l in range(LAYERS)],
                     bv=[vec(5500 + l, KVD) for l in range(LAYERS)])
        for key, name in (("wq", "q"), ("wk", "k"), ("wv", "v"), ("wo", "o"), ("wgate", "gate"), ("wup", "up"),
                          ("wdown", "down")):
            dec_w[key] = [layer_w[l][name] for l in range(LAYERS)]
        cfg = dict(hidden=H, inter=INTER, n_heads=14, n_kv_heads=2, head_dim=64, n_layers=LAYERS, vocab=VOCAB,
                   max_pos=512, rms_eps=1e-6, rope_theta=1000000.0)
        dec = mil.Decoder(cfg, dec_w)
        assert dec.reset(queue, 0, 785)
        assert dec.step(queue)
        queue.finish()
        assert dec.reset(queue, 0, 785)
        with mil.Graph(queue) as step_graph:
            assert dec.step(queue)
        for _ in range(8):
            step_graph.launch()
        ms_tok = time_region(mil, queue, step_graph.launch, 8, 9)
        pos_after, _ = dec.read(queue)
        detail["c4_whole_decode_step_on_device"] = {
            "us_per_token": round(ms_tok * 1e3, 1), "tokens_per_s": round(1e3 / ms_tok, 1),
            "launches_per_step": 24 * 5 + 3, "positions": f"8..{pos_after - 1}", "launch": "hip_graph"}
        dec.close()

        # the same step with block-32 Q4 weights (the LFM2 bundles' format): norm and SwiGLU ride in the
        # exact Q4 GEMV, the lm_head takes the throughput kernel with the argmax in its epilogue
        q4_keep, q4_w = [], dict(dec_w)
        def make_q4(seed, N, K):
            ph, sh = mil.quantize_q4(mil.synth_normal_f16(seed, 0.02, (N, K)))
            pb, sb = mil.Buffer.from_host(ph), mil.Buffer.from_host(sh)
            assert mil.nnopt_register_q4_weight(pb, sb, N, K)
            q4_keep.extend([pb, sb])
            return pb
        shape_of = {n: (N, K) for n, N, K in LAYER_SHAPES}
        for j, (key, name) in enumerate((("wq", "q"), ("wk", "k"), ("wv", "v"), ("wo", "o"), ("wgate", "gate"),
                                         ("wup", "up"), ("wdown", "down"))):
            q4_w[key] = [make_q4(9000 + l * 16 + j, *shape_of[name]) for l in range(LAYERS)]
        q4_w["lm_head"] = make_q4(8999, VOCAB, H)
        dec = mil.Decoder(cfg, q4_w)
        assert dec.reset(queue, 0, 785)
        assert dec.step(queue)
        queue.finish()
        assert dec.reset(queue, 0, 785)
        with mil.Graph(queue) as step_graph_q4:
            assert dec.step(queue)
        for _ in range(8):
            step_graph_q4.launch()
        ms_tok = time_region(mil, queue, step_graph_q4.launch, 8, 9)
        detail["c4_whole_decode_step_on_device_q4_weights"] = {
            "us_per_token": round(ms_tok * 1e3, 1), "tokens_per_s": round(1e3 / ms_tok, 1), "launch": "hip_graph"}
        dec.close()
        for i in range(0, len(q4_keep), 2):
            mil.nnopt_unregister_weight(q4_keep[i])
        del q4_keep, q4_w

    # ---- config 5: prefill GEMM with fused int8 dequant on the matrix cores ---------------
    if not args.no_detail:
        MFMA_PEAK_TFLOPS = 2500.0
        for (N, K) in ((INTER, H), (H, INTER)):
            w = mil.synth_normal_f16(77, 0.02, (N, K))
            qh, sh = mil.quantize_int8(w)
            wb, sb = mil.Buffer.from_host(qh), mil.Buffer.from_host(sh)
            assert mil.nnopt_register_int8_weight(wb, sb, N, K)
            for M in (16, 64, 512, 2048):
                xb = mil.Buffer.from_host(mil.synth_normal_f16(78, 1.0, (M, K)))
                ob = mil.Buffer(M * N * 2)
                arr = mil.make_calls([(M, N, K, xb, wb, ob)] * 20)
                mil.linear_batch(queue, arr)
                ms = time_region(mil, queue, lambda: mil.linear_batch(queue, arr), 1, 9) / 20
                flop = 2.0 * M * N * K
                nbytes = 2 * M * K + N * K + 2 * N + 2 * M * N
                kern, rows, slices = mil.linear_plan(queue, M, N, K, xb, wb)
                detail[f"c5_int8_gemm_M{M}_N{N}_K{K}"] = {
                    "kernel": {1: "wide", 2: "tile64", 3: "tile128", 4: "streaming"}.get(kern, str(kern)),
                    "rows_of_x_per_block": rows, "k_slices": slices,
                    "us": round(ms * 1e3, 2), "TFLOPs": round(flop / (ms * 1e-3) / 1e12, 1),
                    "frac_mfma_fp16_peak": round(flop / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4),
                    "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
            mil.nnopt_unregister_weight(wb)
        # a batch of 16 rows against the lm_head (batched decode): the weights stream once, as for one row
        xb = mil.Buffer.from_host(mil.synth_normal_f16(78, 1.0, (16, H)))
        ob = mil.Buffer(16 * VOCAB * 2)
        arr = mil.make_calls([(16, VOCAB, H, xb, copies[i % 3][0], ob) for i in range(9)])
        mil.linear_batch(queue, arr)
        ms = time_region(mil, queue, lambda: mil.linear_batch(queue, arr), 1, 9) / 9
        nbytes = VOCAB * H + 2 * VOCAB + 2 * 16 * H + 2 * 16 * VOCAB
        detail[f"c5_int8_gemm_M16_N{VOCAB}_K{H}"] = {
            "us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
            "frac_hbm": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        # a large square contraction (no config asks for it): the MFMA main loop without the short K of the
        # configured shapes; the library's own choice (256 x 256 blocks) and the 160-row wide tiles
        Mq = Nq = Kq = 8192
        qh, sh = mil.quantize_int8(mil.synth_normal_f16(79, 0.02, (Nq, Kq)))
        wb, sb = mil.Buffer.from_host(qh), mil.Buffer.from_host(sh)
        assert mil.nnopt_register_int8_weight(wb, sb, Nq, Kq)
        xb = mil.Buffer.from_host(mil.synth_normal_f16(80, 1.0, (Mq, Kq)))
        ob = mil.Buffer(Mq * Nq * 2)
        arr = mil.make_calls([(Mq, Nq, Kq, xb, wb, ob)] * 3)
        for mode, tag in ((0, "proxy_int8_gemm_M8192_N8192_K8192"), (15, "proxy_int8_gemm_M8192_N8192_K8192_160_row_tiles")):
            mil.lib().mi_set_gemm_mode(mode)
            try:
                kern, rows, slices = mil.linear_plan(queue, Mq, Nq, Kq, xb, wb)
                mil.linear_batch(queue, arr)
                ms = time_region(mil, queue, lambda: mil.linear_batch(queue, arr), 1, 5) / 3
            finally:
                mil.lib().mi_set_gemm_mode(0)
            flop = 2.0 * Mq * Nq * Kq
            detail[tag] = {"kernel": {1: "wide", 5: "blocks256"}.get(kern, str(kern)), "rows_of_x_per_block": rows,
                           "us": round(ms * 1e3, 1), "TFLOPs": round(flop / (ms * 1e-3) / 1e12, 1),
                           "frac_mfma_fp16_peak": round(flop / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)}
        mil.nnopt_unregister_weight(wb)
        del xb, ob, wb, sb
        # the same contractions with fp16 weights
        for (N, K) in ((INTER, H), (H, INTER)):
            wb = mil.Buffer.from_host(mil.synth_normal_f16(77, 0.02, (N, K)))
            M = 2048
            xb = mil.Buffer.from_host(mil.synth_normal_f16(78, 1.0, (M, K)))
            ob = mil.Buffer(M * N * 2)
            arr = mil.make_calls([(M, N, K, xb, wb, ob)] * 20)
            mil.linear_batch(queue, arr)
            ms = time_region(mil, queue, lambda: mil.linear_batch(queue, arr), 1, 9) / 20
            flop = 2.0 * M * N * K
            detail[f"c5_fp16_gemm_M{M}_N{N}_K{K}"] = {
                "us": round(ms * 1e3, 2), "TFLOPs": round(flop / (ms * 1e-3) / 1e12, 1),
                "frac_mfma_fp16_peak": round(flop / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)}
        # the same contraction with Q4 weights: exact two-term feed (default) and single rounding (mode 4)
        N, K = INTER, H
        ph, sh = mil.quantize_q4(mil.synth_normal_f16(77, 0.02, (N, K)))
        wb, sb = mil.Buffer.from_host(ph), mil.Buffer.from_host(sh)
        assert mil.nnopt_register_q4_weight(wb, sb, N, K)
        for M in (16, 2048):
            xb = mil.Buffer.from_host(mil.synth_normal_f16(78, 1.0, (M, K)))
            ob = mil.Buffer(M * N * 2)
            arr = mil.make_calls([(M, N, K, xb, wb, ob)] * 20)
            for mode, tag in ((0, "q4"), (4, "q4_single_rounding")):
                mil.lib().mi_set_gemm_mode(mode)
                try:
                    mil.linear_batch(queue, arr)
                    ms = time_region(mil, queue, lambda: mil.linear_batch(queue, arr), 1, 9) / 20
                finally:
                    mil.lib().mi_set_gemm_mode(0)
                flop = 2.0 * M * N * K
                detail[f"c5_{tag}_gemm_M{M}_N{N}_K{K}"] = {
                    "us": round(ms * 1e3, 2), "TFLOPs": round(flop / (ms * 1e-3) / 1e12, 1),
                    "frac_mfma_fp16_peak": round(flop / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)}
        mil.nnopt_unregister_weight(wb)

    # ---- a prompt at once (after the GEMM lines above, which it would otherwise disturb: it
    # allocates and frees a few hundred MB) ----------------------------------------------
    if not args.no_detail and not args.no_graph:
        # a prompt at once: the M-row projections of all 24 layers through the GEMM, the last
        # position's lm_head and argmax; against M single-token steps at the rate measured above
        big = mil.Decoder(dict(cfg, max_pos=2048), dec_w)
        for M in (64, 512, 2048):
            ids = [int(t) for t in np.random.default_rng(M).integers(0, VOCAB, M)]
            assert big.prefill(queue, ids)
            ms = time_region(mil, queue, lambda: big.prefill(queue, ids), 1, 3)
            detail[f"c5_whole_prompt_on_device_M{M}"] = {
                "ms": round(ms, 3), "prompt_tokens_per_s": round(M / ms * 1e3, 0),
                "vs_single_token_steps": round(M * ms_tok / ms, 1)}
        # a decode step at a long context (positions 1900..1931 of the same decoder; the cache's contents do
        # not matter for the time): the reference-order attention and the mode that splits a head's keys
        long_ctx = {"positions": "1900..1931"}
        for name, splits in (("us_per_token_reference_order", 0), ("us_per_token_16_key_splits", 16)):
            assert big.set_attention_splits(splits)
            assert big.reset(queue, 1900, 5) and big.step(queue)
            queue.finish()
            assert big.reset(queue, 1900, 5)
            with mil.Graph(queue) as g:
                assert big.step(queue)

            def run32():
                for _ in range(32):
                    g.launch()
            samples = []
            for _ in range(3):
                assert big.reset(queue, 1900, 5)
                queue.finish()
                samples.append(time_region(mil, queue, run32, 1, 1) / 32)
            long_ctx[name] = round(sorted(samples)[1] * 1e3, 1)
        assert big.set_attention_splits(0)
        detail["c4_decode_step_long_context"] = long_ctx
        big.close()

    # ---- CPU baseline: the oracle on a bounded sample of the same sweep -------------------
    cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle_lib as O
        threads = O.lib.orc_max_threads()
        xh = mil.synth_normal_f16(1, 1.0, (H,))
        xi = mil.synth_normal_f16(2, 1.0, (INTER,))
        sample_bytes, t0, reps = 0, time.time(), 0
        while time.time() - t0 < 12.0 or reps < 2:
            for name, N, K in LAYER_SHAPES:                    # layer 0 of the sweep ...
                q, s = host_layer0[name]
                O.gemv_i8(xi if K == INTER else xh, q, s.view(np.uint16), threads)
                sample_bytes += N * K + 2 * N
            O.gemv_i8(xh, lm_host[0], lm_host[1].view(np.uint16), threads)   # ... and the lm_head
            sample_bytes += VOCAB * H + 2 * VOCAB
            reps += 1
        dt = time.time() - t0
        # per config, beside the GPU figures in `detail`: the same call on the host, all threads
        # and one thread (bounded: each timed for about 0.3 s)
        if not args.no_detail:
            def cpu_us(fn):
                fn()
                t, n = time.time(), 0
                while time.time() - t < 0.3 or n < 1:
                    fn()
                    n += 1
                return round((time.time() - t) / n * 1e6, 1)

            w1 = mil.synth_normal_f16(31, 0.02, (1536, 576))
            x1 = mil.synth_normal_f16(32, 1.0, (576,))
            gq, gs = host_layer0["gate"]
            dq, ds = host_layer0["down"]
            lp, lsc = mil.quantize_q4(mil.synth_normal_f16(7, 0.02, (VOCAB, H)))
            X16 = mil.synth_normal_f16(78, 1.0, (16, H))
            cases = {
                "c1_fp16_gemv_1536x576": lambda t: O.gemv_f16(x1, w1, t),
                "c2_int8_gemv_4864x896": lambda t: O.gemv_i8(xh, gq, gs.view(np.uint16), t),
                "c2_int8_gemv_896x4864": lambda t: O.gemv_i8(xi, dq, ds.view(np.uint16), t),
                "c3_int8_gemv_151936x896": lambda t: O.gemv_i8(xh, lm_host[0], lm_host[1].view(np.uint16), t),
                "c3_q4_gemv_151936x896": lambda t: O.gemv_q4(xh, lp, lsc.view(np.uint16), t),
                "c5_int8_gemm_M16_N4864_K896": lambda t: O.gemm_i8(X16, gq, gs.view(np.uint16), t),
            }
            detail["cpu_port"] = {"cores": threads}
            for name, fn in cases.items():
                detail["cpu_port"][name] = {"us_all_cores": cpu_us(lambda: fn(threads)),
                                            "us_one_core": cpu_us(lambda: fn(1))}
        cpu_model, cpu_allowed, cpu_online = host_cpu()
        cpu = {"value": round(sample_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
               "compiler_flags": O.lib.orc_build_flags().decode(),
               "cpu_model": cpu_model, "cores_in_affinity_mask": cpu_allowed, "cores_online": cpu_online,
               "sample": f"{reps} x (layer 0's 7 int8 GEMVs + the lm_head GEMV), {sample_bytes} algorithmic "
                         f"bytes in {dt:.1f} s, OpenMP over rows"}

    out = {
        "metric": "quant GEMV achieved HBM GB/s (% of peak) + us/decode-step, Qwen2.5-0.5B shapes",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",          # the sums; operands: int8 weights and fp16 scales, fp16 activations
        "config": {"workload": "Qwen2.5-0.5B decode-step matmul sweep, batch 1, per-row int8: 24 x "
                               "{q,k,v,o,gate,up,down} + lm_head = 169 GEMVs, 494873344 algorithmic bytes",
                   "operands": "int8 weights with fp16 row scales, fp16 activations and outputs, fp32 accumulate",
                   "launch": launch_mode, "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                   "us_per_decode_step": round(ms_step * 1e3, 1)},
        "roofline": roofline, "cpu_baseline": cpu, "detail": detail,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
