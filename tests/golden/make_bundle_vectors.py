"""Writes tests/golden/bundle/*: a tiny synthetic fp16 weight bundle and what the reference's own
bundle quantisers make of it (int8 and q4, with and without the embedding options).

Runs in the build container only (it executes /root/reference/src/models/lfm2-5-350m/scripts/
quantize_weights.py and quantize_q4.py as command-line tools); the files it writes are the
fixtures, a few KB each.  The file layout these tools produce (order, offsets, meta fields, the
lm_head alias) is not covered by any other fixture of the reference.
"""
import importlib
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "bundle")
REF = "/root/reference/src/models/lfm2-5-350m/scripts"


def main():
    sys.path.insert(0, ROOT)
    bt = importlib.import_module("adreno-llms_amd.bundle_tools")
    rng = np.random.default_rng(20240607)

    def w(*shape, scale=0.02):
        return (rng.standard_normal(shape) * scale).astype(np.float16)

    tensors = {
        "model.embed_tokens.weight": w(40, 64),
        "model.embedding_norm.weight": (1.0 + w(64)).astype(np.float16),
        "model.layers.0.conv.conv.weight": w(64, 1, 3, scale=0.3),           # 3-D: passes through
        "model.layers.0.conv.in_proj.weight": w(48, 64),
        "model.layers.0.conv.out_proj.weight": w(16, 64),
        "model.layers.0.feed_forward.w1.weight": w(24, 64),
        "model.layers.0.feed_forward.w2.weight": w(64, 96),                   # K = 96: three q4 blocks per row
        "model.layers.0.feed_forward.w3.weight": w(24, 64),
        "model.layers.0.operator_norm.weight": (1.0 + w(64)).astype(np.float16),
        "model.layers.1.self_attn.q_proj.weight": w(16, 64),
        "model.layers.1.self_attn.k_proj.weight": w(8, 64),
        "model.layers.1.self_attn.v_proj.weight": w(8, 64),
        "model.layers.1.self_attn.out_proj.weight": w(16, 64),
        "model.layers.1.self_attn.q_layernorm.weight": (1.0 + w(16)).astype(np.float16),
    }
    tensors["model.layers.1.self_attn.k_proj.weight"][3] = 0            # an all-zero row and block
    tensors["model.layers.0.conv.in_proj.weight"][5, 7] = np.float16(0.75)   # an outlier that sets its row's scale
    os.makedirs(OUT, exist_ok=True)
    fp16_bin, fp16_meta = os.path.join(OUT, "tiny.fp16.bin"), os.path.join(OUT, "tiny.fp16.meta.json")
    bt.write_fp16_bundle(tensors, fp16_bin, fp16_meta, model_id="synthetic/tiny-lfm2")

    runs = [
        ("quantize_weights.py", "int8", []),
        ("quantize_weights.py", "int8_embed_alias", ["--quantize-embed", "--emit-lm-head-int8"]),
        ("quantize_q4.py", "q4", []),
        ("quantize_q4.py", "q4_alias", ["--emit-lm-head-q4"]),
    ]
    for script, tag, extra in runs:
        cmd = [sys.executable, os.path.join(REF, script), "--fp16-bin", fp16_bin, "--fp16-meta", fp16_meta,
               "--out-bin", os.path.join(OUT, f"tiny.{tag}.bin"),
               "--out-meta", os.path.join(OUT, f"tiny.{tag}.meta.json"), *extra]
        subprocess.check_call(cmd)
    for f in sorted(os.listdir(OUT)):
        print(f, os.path.getsize(os.path.join(OUT, f)))


if __name__ == "__main__":
    main()
