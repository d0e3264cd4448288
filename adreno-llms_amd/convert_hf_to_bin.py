"""safetensors checkpoint -> fp16 weight bundle (`model.fp16.bin` + `model.fp16.meta.json`), the
first step of the reference's weight pipeline (scripts/convert_hf_to_bin.py), with the same
command line, the same files byte for byte, and the same `--check-against` report.

Container format read here (scripts/convert_hf_to_bin.py:42-65): 8 bytes little-endian header
length n, n bytes of JSON {name: {dtype, shape, data_offsets: [begin, end)}} (+ an optional
"__metadata__" entry), then the tensor bytes, offsets counted from the end of the header.  A
directory is read through `model.safetensors.index.json` when present (only the shards its
weight_map names), else every `*.safetensors` in it (scripts/convert_hf_to_bin.py:68-95).
Every tensor becomes fp16: F64 / F32 / F16 and the integer types by one rounding from their own
value, BF16 by placing its 16 bits in the upper half of an fp32 (exact) and rounding that
(scripts/convert_hf_to_bin.py:42-57, 98-106).  Tensors are laid out in sorted-name order with no
padding; the meta entry of each is {offset, shape, dtype "float16", num_elements, size_bytes}
(scripts/convert_hf_to_bin.py:149-170).

Unlike the reference this streams: the layout is computed from the headers alone, and tensors
are converted one at a time from a memory map, so a checkpoint never has to fit in memory twice.

  python convert_hf_to_bin.py --input DIR_OR_FILE [--model-id ID] [--output-dir OUT]
                              [--check-against META.json]
"""
import argparse
import json
import os
import struct
import sys

import numpy as np

# safetensors dtype -> (little-endian numpy dtype of the stored bytes, bytes per element)
DTYPES = {
    "F64": "<f8", "F32": "<f4", "F16": "<f2", "BF16": "<u2",
    "I64": "<i8", "I32": "<i4", "I16": "<i2", "I8": "<i1", "U8": "<u1", "BOOL": "<u1",
}
INDEX_NAME = "model.safetensors.index.json"


class ConvertError(SystemExit):
    """Raised with the `ERROR: ...` text the reference tool exits with."""

    def __init__(self, msg):
        super().__init__(f"ERROR: {msg}")


def read_header(path):
    """-> (entries without __metadata__, offset of the first tensor byte)."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    header.pop("__metadata__", None)
    return header, 8 + n


def shard_files(input_path):
    """The .safetensors files an --input names, sorted, each once."""
    if os.path.isfile(input_path):
        if not input_path.endswith(".safetensors"):
            raise ConvertError(f"{input_path} is not a .safetensors file")
        return [input_path]
    if not os.path.isdir(input_path):
        raise ConvertError(f"--input not found: {input_path}")
    index = os.path.join(input_path, INDEX_NAME)
    if os.path.exists(index):
        with open(index, encoding="utf-8") as f:
            names = set(json.load(f)["weight_map"].values())
    else:
        names = {f for f in os.listdir(input_path) if f.endswith(".safetensors")}
        if not names:
            raise ConvertError(f"no .safetensors found under {input_path}")
    return sorted(os.path.join(input_path, n) for n in names)


class Tensor:
    __slots__ = ("name", "path", "begin", "end", "dtype", "shape", "count")

    def __init__(self, name, path, data_start, info):
        if info["dtype"] not in DTYPES:
            raise ConvertError(f"{name}: unsupported dtype {info['dtype']}")
        self.name, self.path, self.dtype = name, path, info["dtype"]
        self.begin, self.end = data_start + info["data_offsets"][0], data_start + info["data_offsets"][1]
        self.shape = list(info["shape"])
        self.count = int(np.prod(self.shape)) if self.shape else 1
        stored = (self.end - self.begin) // np.dtype(DTYPES[self.dtype]).itemsize
        if stored != self.count:
            raise ConvertError(f"{name}: element count {stored} != prod(shape) {self.count}")

    def fp16(self, maps):
        """The tensor's values as a flat fp16 array."""
        raw = maps(self.path)[self.begin:self.end]
        a = np.frombuffer(raw, dtype=DTYPES[self.dtype])
        if self.dtype == "BF16":
            a = (a.astype(np.uint32) << 16).view(np.float32)
        with np.errstate(over="ignore", invalid="ignore"):
            return a.astype(np.float16)


def scan(input_path):
    """Sorted list of Tensor for everything under input_path; reads headers only."""
    found = {}
    for path in shard_files(input_path):
        header, data_start = read_header(path)
        for name, info in header.items():
            if name in found:
                raise ConvertError(f"tensor {name!r} present in multiple shards")
            found[name] = Tensor(name, path, data_start, info)
    return [found[n] for n in sorted(found)]


def make_meta(model_id, tensors):
    """The meta.json object of an fp16 bundle (scripts/convert_hf_to_bin.py:149-170)."""
    offset, entries = 0, {}
    for t in tensors:
        size = 2 * t.count
        entries[t.name] = {"offset": offset, "shape": t.shape, "dtype": "float16",
                           "num_elements": t.count, "size_bytes": size}
        offset += size
    return {"model_id": model_id, "format": "binary", "layout": "row_major", "dtype": "float16",
            "quantization": {"enabled": True, "bits": 16, "method": "float16"},
            "total_bytes": offset, "tensors": entries}


def check_against(meta, ref_path, out=sys.stdout):
    """Diff of the generated layout against an existing meta.json, one line per difference in
    the reference tool's wording (scripts/convert_hf_to_bin.py:172-192).  Returns the count."""
    with open(ref_path, encoding="utf-8") as f:
        ref = json.load(f)
    gen_t, ref_t = meta["tensors"], ref["tensors"]
    lines = [f"  + generated has extra tensor: {k}" for k in sorted(set(gen_t) - set(ref_t))]
    lines += [f"  - reference has tensor not generated: {k}" for k in sorted(set(ref_t) - set(gen_t))]
    for k in sorted(set(gen_t) & set(ref_t)):
        lines += [f"  ~ {k}.{field}: gen={gen_t[k][field]} ref={ref_t[k][field]}"
                  for field in ("offset", "shape", "size_bytes", "num_elements")
                  if gen_t[k][field] != ref_t[k][field]]
    if meta["total_bytes"] != ref["total_bytes"]:
        lines.append(f"  ~ total_bytes: gen={meta['total_bytes']} ref={ref['total_bytes']}")
    for line in lines:
        print(line, file=out)
    return len(lines)


class _Maps:
    """One read-only memory map per shard, opened on first use."""

    def __init__(self):
        self._m = {}

    def __call__(self, path):
        if path not in self._m:
            self._m[path] = np.memmap(path, dtype=np.uint8, mode="r")
        return self._m[path]


def convert(input_path, output_dir=None, model_id=None, check=None, out=sys.stdout):
    """Runs the tool; returns its exit status (0 ok, 1 mismatch without --output-dir or a short write)."""
    model_id = model_id or os.path.basename(os.path.abspath(input_path))
    print(f"Reading: {input_path}", file=out)
    tensors = scan(input_path)
    meta = make_meta(model_id, tensors)
    print(f"Layout: {len(tensors)} tensors, {meta['total_bytes']:,} bytes (fp16)", file=out)
    if check:
        print(f"Checking against {check} ...", file=out)
        diffs = check_against(meta, check, out)
        if diffs:
            print(f"MISMATCH: {diffs} difference(s) ✗", file=out)
            if not output_dir:
                return 1
        else:
            print("MATCH: generated layout is byte-identical ✓", file=out)
    if output_dir:
        os.makedirs(output_dir, exist_ok=True)
        bin_path = os.path.join(output_dir, "model.fp16.bin")
        meta_path = os.path.join(output_dir, "model.fp16.meta.json")
        maps = _Maps()
        with open(bin_path, "wb") as f:
            for t in tensors:
                f.write(memoryview(np.ascontiguousarray(t.fp16(maps))).cast("B"))
        with open(meta_path, "w", encoding="utf-8") as f:
            json.dump(meta, f, indent=2)
        written = os.path.getsize(bin_path)
        if written != meta["total_bytes"]:
            print(f"ERROR: wrote {written} bytes, expected {meta['total_bytes']}", file=sys.stderr)
            return 1
        print(f"Wrote {bin_path} ({written:,} bytes) ✓", file=out)
        print(f"Wrote {meta_path} ✓", file=out)
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(description="safetensors checkpoint -> fp16 weight bundle")
    ap.add_argument("--input", default=None, help="a .safetensors file or a model directory (sharded or not)")
    ap.add_argument("--hf-repo-id", default=None,
                    help="not supported here: fetch the checkpoint yourself and pass --input")
    ap.add_argument("--model-id", default=None, help="label stored in meta.json (default: basename of --input)")
    ap.add_argument("--output-dir", default=None, help="where model.fp16.bin and model.fp16.meta.json go")
    ap.add_argument("--check-against", default=None, metavar="META",
                    help="compare the generated layout with an existing meta.json; writes nothing "
                         "unless --output-dir is given as well")
    a = ap.parse_args(argv)
    if a.hf_repo_id or not a.input:
        print("ERROR: pass --input (a local .safetensors file or directory); downloading is not part "
              "of this tool", file=sys.stderr)
        return 1
    return convert(a.input, a.output_dir, a.model_id, a.check_against)


if __name__ == "__main__":
    sys.exit(main())
