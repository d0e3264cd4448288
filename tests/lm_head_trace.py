"""Runs the lm_head GEMV (151 936 x 896) as stream launches, rotating through weight copies larger
than the last-level cache: Q4 with the throughput kernel (gemv mode 1), Q4 in the reference's order
(mode 0), int8, and the streaming-read probe over the same bytes.  The program behind the counter
summaries of these kernels in profiles/ (a profile needs launches, not a graph replay)."""
import importlib, os, sys

import numpy as np
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
mil = importlib.import_module("adreno-llms_amd")
assert mil.lib().mi_init(0) == 1
queue = mil.Queue()
N, K, REPS = 151936, 896, int(sys.argv[1]) if len(sys.argv) > 1 else 40
w = mil.synth_normal_f16(7, 0.02, (N, K))
x = mil.Buffer.from_host(mil.synth_normal_f16(1, 1.0, (K,)))
y = mil.Buffer(N * 2)
p, sc = mil.quantize_q4(w)
q, s = mil.quantize_int8(w)
q4 = [(mil.Buffer.from_host(p), mil.Buffer.from_host(sc)) for _ in range(4)]      # 4 x 77 MB
i8 = [(mil.Buffer.from_host(q), mil.Buffer.from_host(s)) for _ in range(3)]       # 3 x 136 MB
for wb, sb in q4:
    assert mil.nnopt_register_q4_weight(wb, sb, N, K)
for wb, sb in i8:
    assert mil.nnopt_register_int8_weight(wb, sb, N, K)


def timed(fn, n):
    e0, e1 = mil.Event(), mil.Event()
    fn(0)
    queue.finish()
    e0.record(queue)
    for i in range(n):
        fn(i)
    e1.record(queue)
    e1.synchronize()
    return e0.elapsed_ms(e1) / n * 1e3


for mode in (1, 0):
    mil.lib().mi_set_gemv_mode(mode)
    us = timed(lambda i: mil.pytorch_linear(queue, 1, N, K, x, q4[i % 4][0], y), REPS)
    print(f"q4 lm_head, gemv mode {mode}: {us:.2f} us per launch", flush=True)
mil.lib().mi_set_gemv_mode(1)
us = timed(lambda i: mil.pytorch_linear(queue, 1, N, K, x, i8[i % 3][0], y), REPS)
print(f"int8 lm_head: {us:.2f} us per launch", flush=True)
q4_bytes = (N * K // 2 + N * (K // 32) * 2) // 16 * 16
us = timed(lambda i: mil.lib().mi_stream_read_probe(queue.handle, i8[i % 3][0].ptr, q4_bytes, None), REPS)
print(f"read probe, {q4_bytes} bytes (a Q4 lm_head's): {us:.2f} us per launch", flush=True)
us = timed(lambda i: mil.lib().mi_stream_read_probe(queue.handle, i8[i % 3][0].ptr, N * K, None), REPS)
print(f"read probe, {N * K} bytes (an int8 lm_head's): {us:.2f} us per launch", flush=True)
queue.finish()
