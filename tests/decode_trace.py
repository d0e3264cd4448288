"""Runs greedy steps of the device decoder on Qwen2.5-0.5B shapes as stream launches: the program behind
profiles/decode_step_kernel_trace.txt (a kernel trace needs launches, not a graph replay).
No arguments: 63 steps from position 0.  `decode_trace.py POS SPLITS`: 16 steps from position POS of a decoder
for 2048 positions (the cache's contents do not matter for the time), the attention in the reference's order
(SPLITS = 0) or with a head's keys split over SPLITS blocks: profiles/decode_step_long_context_kernel_trace.txt."""
import importlib, os, sys

import numpy as np
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT); sys.path.insert(0, os.path.join(ROOT, "tests"))
mil = importlib.import_module("adreno-llms_amd")
from decode_harness import PROMPT, QWEN25_05B, GpuDecoder, Model
assert mil.lib().mi_init(0) == 1
queue = mil.Queue()
if len(sys.argv) > 2:
    pos0, splits = int(sys.argv[1]), int(sys.argv[2])
    m = Model(dict(QWEN25_05B, max_pos=2048), seed=2024)
    gd = GpuDecoder(m, queue)
    assert gd.dec.set_attention_splits(splits)
    assert gd.dec.reset(queue, pos0, 5)
    for _ in range(16):
        assert gd.dec.step(queue)
    queue.finish()
    print("done", gd.dec.read(queue), flush=True)
else:
    m = Model(QWEN25_05B, seed=2024)
    gd = GpuDecoder(m, queue)
    toks = gd.greedy(PROMPT, 58, graph=False)
    print("done", toks[:4], flush=True)
gd.close()
