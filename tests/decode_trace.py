"""Runs 63 greedy steps of the device decoder on Qwen2.5-0.5B shapes as stream launches: the program
behind profiles/decode_step_kernel_trace.txt (a kernel trace needs launches, not a graph replay)."""
import importlib, os, sys

import numpy as np
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT); sys.path.insert(0, os.path.join(ROOT, "tests"))
mil = importlib.import_module("adreno-llms_amd")
from decode_harness import PROMPT, QWEN25_05B, GpuDecoder, Model
assert mil.lib().mi_init(0) == 1
queue = mil.Queue()
m = Model(QWEN25_05B, seed=2024)
gd = GpuDecoder(m, queue)
toks = gd.greedy(PROMPT, 58, graph=False)
print("done", toks[:4], flush=True)
gd.close()
