"""Writes tests/golden/convert/*: two synthetic safetensors checkpoints (one file; a directory of
two shards with an index and a stray file the index does not name) and what the reference's own
converter makes of them: the fp16 bundle, its meta.json, and the text of its --check-against
report against a meta.json with one difference of every kind.

Runs in the build container only (it executes /root/reference/scripts/convert_hf_to_bin.py as a
command-line tool with --input); the files it writes are the fixtures, a few KB each.  No other
fixture of the reference covers the container parsing, the dtype table, the shard handling or
the report format.
"""
import json
import os
import struct
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "convert")
REF = "/root/reference/scripts/convert_hf_to_bin.py"

CODES = {np.dtype("<f8"): "F64", np.dtype("<f4"): "F32", np.dtype("<f2"): "F16", np.dtype("<i8"): "I64",
         np.dtype("<i4"): "I32", np.dtype("<i2"): "I16", np.dtype("<i1"): "I8", np.dtype("<u1"): "U8"}


def write_safetensors(path, tensors, metadata=None):
    """tensors: list of (name, dtype code or None, array, shape or None) in file order."""
    header, blobs, off = {}, [], 0
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, code, arr, shape in tensors:
        arr = np.ascontiguousarray(arr)
        raw = arr.tobytes()
        header[name] = {"dtype": code or CODES[arr.dtype], "shape": list(arr.shape if shape is None else shape),
                        "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)                     # the format pads the header with spaces
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for b in blobs:
            f.write(b)


def bf16_bits(values):
    """fp32 values truncated to their upper 16 bits."""
    return (np.asarray(values, np.float32).view(np.uint32) >> 16).astype("<u2")


def main():
    os.makedirs(OUT, exist_ok=True)
    rng = np.random.default_rng(20250101)
    n = lambda *s, scale=0.02: rng.standard_normal(s) * scale

    # bf16 patterns chosen for the second rounding: exact fp16 values, halfway cases (the 8 bits of
    # a bf16 mantissa fit fp16's 10, so ties only arise in the subnormal range and at overflow),
    # fp16 subnormals, values below the smallest subnormal, above the largest finite, inf, nan, -0
    bf_special = np.array([0.0, -0.0, 1.0, -1.5, 65280.0, 65536.0, 1e38, -1e38, np.inf, -np.inf, np.nan,
                           2.0 ** -14, 2.0 ** -15, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 2.0 ** -26,
                           -3.0 * 2.0 ** -25, 0.33203125, 3.140625], np.float32)
    f32_special = np.array([65504.0, 65519.9, 65520.0, 1e6, -1e6, 2049.0, 2051.0, 1e-8, 6e-8, 3e-8,
                            2.98023224e-08, -2.98023224e-08, np.float32(np.pi), 0.1], np.float32)
    single = [   # written in this (unsorted) order; the bundle must come out sorted by name
        ("model.norm.weight", None, (1.0 + n(16)).astype("<f4"), None),
        ("model.layers.0.self_attn.q_proj.weight", "BF16", bf16_bits(n(8, 16)), (8, 16)),
        ("model.layers.0.self_attn.q_proj.bias", "BF16", bf16_bits(bf_special), (bf_special.size,)),
        ("model.embed_tokens.weight", None, n(12, 16).astype("<f2"), None),
        ("model.layers.0.mlp.down_proj.weight", None, n(16, 24).astype("<f8"), None),
        ("model.layers.0.conv.weight", None, n(4, 1, 3, scale=0.3).astype("<f4"), None),
        ("lm_head.scalar", None, np.array(0.7071067811865476, "<f8"), ()),
        ("extras.f32_edge", None, f32_special.astype("<f4"), None),
        ("extras.i64", None, np.array([0, 1, -1, 2047, 2049, 65504, 70000, -(2 ** 40)], "<i8"), None),
        ("extras.i32", None, np.array([[3, -4], [2048, -2051]], "<i4"), None),
        ("extras.i16", None, np.array([-32768, 32767, 5], "<i2"), None),
        ("extras.i8", None, np.array([-128, 127, 0, -1], "<i1"), None),
        ("extras.u8", None, np.array([0, 255, 128], "<u1"), None),
        ("extras.bool", "BOOL", np.array([1, 0, 1, 1], "<u1"), None),
        ("Zeta.first_in_ascii_order", None, n(5).astype("<f2"), None),   # upper case sorts before lower
    ]
    write_safetensors(os.path.join(OUT, "single.safetensors"), single, metadata={"format": "pt"})

    shard_dir = os.path.join(OUT, "sharded")
    os.makedirs(shard_dir, exist_ok=True)
    a = [("model.layers.1.w", "BF16", bf16_bits(n(6, 8)), (6, 8)),
         ("model.embed_tokens.weight", None, n(10, 8).astype("<f4"), None)]
    b = [("model.layers.0.w", None, n(6, 8).astype("<f2"), None),
         ("model.norm.weight", "BF16", bf16_bits(1.0 + n(8)), (8,)),
         ("model.layers.10.w", None, n(2, 8).astype("<f4"), None)]       # "10" sorts before "1." ... as text
    write_safetensors(os.path.join(shard_dir, "model-00001-of-00002.safetensors"), a, metadata={"format": "pt"})
    write_safetensors(os.path.join(shard_dir, "model-00002-of-00002.safetensors"), b)
    write_safetensors(os.path.join(shard_dir, "consolidated.safetensors"),
                      [("model.norm.weight", None, n(8).astype("<f4"), None)])   # not in the index: ignored
    weight_map = {name: "model-00001-of-00002.safetensors" for name, *_ in a}
    weight_map.update({name: "model-00002-of-00002.safetensors" for name, *_ in b})
    with open(os.path.join(shard_dir, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"total_size": 0}, "weight_map": weight_map}, f, indent=1)

    for tag, inp, mid in (("single", os.path.join(OUT, "single.safetensors"), "synthetic/single"),
                          ("sharded", shard_dir, None)):
        dst = os.path.join(OUT, f"{tag}.bundle")
        subprocess.check_call([sys.executable, REF, "--input", inp, "--output-dir", dst]
                              + (["--model-id", mid] if mid else []))

    # --check-against: a reference meta with a missing tensor, an extra one, a changed shape, offset,
    # size and element count, and another total; the tool's report is the fixture
    with open(os.path.join(OUT, "single.bundle", "model.fp16.meta.json")) as f:
        meta = json.load(f)
    t = meta["tensors"]
    del t["extras.u8"]
    t["only.in.reference"] = {"offset": 0, "shape": [1], "dtype": "float16", "num_elements": 1, "size_bytes": 2}
    t["model.norm.weight"]["shape"] = [4, 4]
    t["model.embed_tokens.weight"]["offset"] += 2
    t["extras.i8"]["size_bytes"] = 10
    t["extras.i8"]["num_elements"] = 5
    meta["total_bytes"] += 6
    other = os.path.join(OUT, "single.other.meta.json")
    with open(other, "w") as f:
        json.dump(meta, f, indent=2)
    for tag, against in (("mismatch", other), ("match", os.path.join(OUT, "single.bundle", "model.fp16.meta.json"))):
        r = subprocess.run([sys.executable, REF, "--input", os.path.join(OUT, "single.safetensors"),
                            "--check-against", against], capture_output=True, text=True)
        text = r.stdout.replace(OUT + os.sep, "")            # paths relative to the fixture folder
        with open(os.path.join(OUT, f"single.check_{tag}.txt"), "w") as f:
            f.write(f"exit {r.returncode}\n{text}")
    for root, _, files in os.walk(OUT):
        for name in sorted(files):
            p = os.path.join(root, name)
            print(os.path.relpath(p, OUT), os.path.getsize(p))


if __name__ == "__main__":
    main()
