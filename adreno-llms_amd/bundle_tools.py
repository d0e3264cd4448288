"""Weight-bundle writers: the `.bin` + `meta.json` pairs this library's loader (and the
reference's `Weights` class, QW/src/weights.cpp:22-140) read.

A bundle is the concatenation of its tensors in sorted-name order without padding, described by
a JSON object with one entry per tensor: {offset, shape, dtype, num_elements, size_bytes}
(scripts/convert_hf_to_bin.py:149-170).  A quantised bundle keeps every name; a quantised tensor
`<name>` (dtype "int8", or "q4_packed" with shape [N, K/2]) is immediately followed by
`<name>.scale` (fp16 [N], or [N, K/32]), everything else passes through as fp16
(LF/scripts/quantize_weights.py:108-175, LF/scripts/quantize_q4.py:124-199).  The optional
lm_head alias is a quantised copy of model.embed_tokens.weight appended under the name
lm_head.weight while the embedding itself stays fp16 for the lookup
(LF/scripts/quantize_weights.py:177-208, LF/scripts/quantize_q4.py:201-230).

The row quantisers are the library's host routines (mi_quantize_int8 / mi_quantize_q4, threaded
C++), so a bundle of a 0.5 B-parameter model converts in seconds; output is byte-identical to the
reference scripts' (tests/test_bundle_tools.py against files those scripts wrote).

Command line:
  python bundle_tools.py int8|q4 --fp16-bin A.bin --fp16-meta A.meta.json --out-bin B.bin \
         --out-meta B.meta.json [--suffix S ...] [--quantize-embed] [--emit-lm-head]
"""
import argparse
import importlib
import json
import os
import sys

import numpy as np

EMBED = "model.embed_tokens.weight"
LM_HEAD = "lm_head.weight"

# nn.Linear weights of the LFM2.5 blocks, the default selection (LF/scripts/quantize_weights.py:28-38);
# other models pass their own suffixes.
LFM2_LINEAR_SUFFIXES = (
    ".self_attn.q_proj.weight", ".self_attn.k_proj.weight", ".self_attn.v_proj.weight",
    ".self_attn.out_proj.weight", ".conv.in_proj.weight", ".conv.out_proj.weight",
    ".feed_forward.w1.weight", ".feed_forward.w2.weight", ".feed_forward.w3.weight",
)


def _lib():
    here = os.path.dirname(os.path.abspath(__file__))
    parent, pkg = os.path.dirname(here), os.path.basename(here)
    if parent not in sys.path:
        sys.path.insert(0, parent)
    return importlib.import_module(pkg)


class BundleWriter:
    """Appends tensors to a .bin in the order given and keeps the running meta entries."""

    def __init__(self, bin_path):
        self._f = open(bin_path, "wb")
        self.offset = 0
        self.tensors = {}

    def add(self, name, data, shape, dtype):
        data = np.ascontiguousarray(data)
        self.tensors[name] = {
            "offset": self.offset,
            "shape": [int(v) for v in shape],
            "dtype": dtype,
            "num_elements": int(np.prod(shape, dtype=np.int64)) if len(shape) else 1,
            "size_bytes": int(data.nbytes),
        }
        self._f.write(data.tobytes() if data.nbytes < (1 << 20) else memoryview(data).cast("B"))
        self.offset += int(data.nbytes)

    def close(self):
        self._f.close()


def write_fp16_bundle(tensors, bin_path, meta_path, model_id=None):
    """tensors: {name: array}; written as fp16 in sorted-name order (scripts/convert_hf_to_bin.py:149-170)."""
    w = BundleWriter(bin_path)
    for name in sorted(tensors):
        a = np.asarray(tensors[name])
        w.add(name, a.astype(np.float16), a.shape, "float16")
    w.close()
    meta = {
        "model_id": model_id, "format": "binary", "layout": "row_major", "dtype": "float16",
        "quantization": {"enabled": True, "bits": 16, "method": "float16"},
        "total_bytes": w.offset, "tensors": w.tensors,
    }
    with open(meta_path, "w") as f:
        f.write(json.dumps(meta, indent=2))
    return meta


def quantize_bundle(scheme, fp16_bin, fp16_meta, out_bin, out_meta, suffixes=LFM2_LINEAR_SUFFIXES,
                    quantize_embed=False, emit_lm_head=False, method=None):
    """fp16 bundle -> int8 (per-row symmetric) or q4 (block-32 symmetric, nibble-packed) bundle.

    scheme: "int8" or "q4".  A tensor is quantised when it is 2-D and its name ends in one of
    `suffixes` (or is the embedding and quantize_embed is set).  Returns the meta dict written."""
    if scheme not in ("int8", "q4"):
        raise ValueError(f"scheme must be 'int8' or 'q4', got {scheme!r}")
    mil = _lib()
    with open(fp16_meta) as f:
        meta = json.load(f)
    tensors_in = meta["tensors"]
    raw = np.memmap(fp16_bin, dtype=np.uint8, mode="r")

    def rows_of(name):
        t = tensors_in[name]
        if t["dtype"] != "float16":
            raise RuntimeError(f"Expected float16 input, got {t['dtype']} for {name}")
        if t["offset"] + t["size_bytes"] > raw.size:
            raise RuntimeError(f"Tensor {name} out of range")
        return raw[t["offset"]:t["offset"] + t["size_bytes"]].view(np.float16)

    def selected(name, shape):
        if len(shape) != 2:
            return False
        if quantize_embed and name == EMBED:
            return True
        return any(name.endswith(s) for s in suffixes)

    def add_quantised(w, name, arr, n, k):
        if scheme == "int8":
            q, s = mil.quantize_int8(arr.reshape(n, k))
            w.add(name, q, (n, k), "int8")
            w.add(name + ".scale", s, (n,), "float16")
        else:
            if k % 32:
                raise RuntimeError(f"{name}: K={k} not divisible by 32")
            p, s = mil.quantize_q4(arr.reshape(n, k))
            w.add(name, p, (n, k // 2), "q4_packed")
            w.add(name + ".scale", s, (n, k // 32), "float16")

    w = BundleWriter(out_bin)
    for name in sorted(tensors_in):
        shape = tensors_in[name]["shape"]
        arr = rows_of(name)
        if selected(name, shape):
            add_quantised(w, name, arr, shape[0], shape[1])
        else:
            w.add(name, arr, shape, "float16")
    alias = False
    if emit_lm_head:
        t = tensors_in.get(EMBED)
        if t is None or t["dtype"] != "float16":
            print(f"warn: the lm_head alias needs an fp16 {EMBED}", file=sys.stderr)
        else:
            add_quantised(w, LM_HEAD, rows_of(EMBED), t["shape"][0], t["shape"][1])
            alias = True
    w.close()

    if scheme == "int8":
        quant = {"enabled": True, "bits": 8,
                 "method": method or "per-row symmetric int8 + fp16 scales; other tensors fp16",
                 "quantized_embed": bool(quantize_embed), "lm_head_int8_alias": alias}
    else:
        quant = {"enabled": True, "bits": 4, "block_size": 32,
                 "method": method or "block-32 symmetric q4: scale = absmax / 7, stored nibble = q + 8, "
                                     "two nibbles per byte (low nibble first); other tensors fp16",
                 "quantized_embed": bool(quantize_embed), "lm_head_q4_alias": alias}
    out = {"model_id": meta.get("model_id"), "format": "binary", "layout": "row_major", "dtype": "mixed",
           "quantization": quant, "tensors": w.tensors}
    with open(out_meta, "w") as f:
        f.write(json.dumps(out, indent=2))
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description="fp16 weight bundle -> int8 / q4 weight bundle")
    ap.add_argument("scheme", choices=("int8", "q4"))
    ap.add_argument("--fp16-bin", required=True)
    ap.add_argument("--fp16-meta", required=True)
    ap.add_argument("--out-bin", required=True)
    ap.add_argument("--out-meta", required=True)
    ap.add_argument("--suffix", action="append", default=None,
                    help="name suffix of 2-D tensors to quantise (repeatable); default: the LFM2.5 linear layers")
    ap.add_argument("--quantize-embed", action="store_true")
    ap.add_argument("--emit-lm-head", action="store_true",
                    help="append a quantised copy of the embedding as lm_head.weight")
    a = ap.parse_args(argv)
    out = quantize_bundle(a.scheme, a.fp16_bin, a.fp16_meta, a.out_bin, a.out_meta,
                          suffixes=tuple(a.suffix) if a.suffix else LFM2_LINEAR_SUFFIXES,
                          quantize_embed=a.quantize_embed, emit_lm_head=a.emit_lm_head)
    nq = sum(1 for t in out["tensors"].values() if t["dtype"] in ("int8", "q4_packed"))
    print(f"{a.out_bin}: {len(out['tensors'])} tensors, {nq} quantised", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
