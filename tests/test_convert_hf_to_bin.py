"""The safetensors -> fp16 bundle converter (adreno-llms_amd/convert_hf_to_bin.py) against files the
reference's own scripts/convert_hf_to_bin.py wrote from the same synthetic checkpoints
(tests/golden/convert/, made by tests/golden/make_convert_vectors.py), plus what the format fixes."""
import importlib
import io
import json
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

cv = importlib.import_module("adreno-llms_amd.convert_hf_to_bin")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
G = os.path.join(ROOT, "tests", "golden", "convert")


def run(inp, **kw):
    out = io.StringIO()
    rc = cv.convert(inp, out=out, **kw)
    return rc, out.getvalue()


@pytest.mark.parametrize("tag,inp,model_id", [("single", "single.safetensors", "synthetic/single"),
                                              ("sharded", "sharded", None)])
def test_bundle_is_byte_identical_to_the_reference_tools_output(tmp_path, tag, inp, model_id):
    rc, text = run(os.path.join(G, inp), output_dir=str(tmp_path), model_id=model_id)
    assert rc == 0
    want_bin = open(os.path.join(G, f"{tag}.bundle", "model.fp16.bin"), "rb").read()
    want_meta = open(os.path.join(G, f"{tag}.bundle", "model.fp16.meta.json")).read()
    assert open(tmp_path / "model.fp16.bin", "rb").read() == want_bin
    assert open(tmp_path / "model.fp16.meta.json").read() == want_meta
    meta = json.loads(want_meta)
    assert list(meta["tensors"]) == sorted(meta["tensors"])
    assert f"Layout: {len(meta['tensors'])} tensors, {meta['total_bytes']:,} bytes (fp16)" in text


def test_a_directory_without_index_takes_every_safetensors_file(tmp_path):
    # without the index the stray third file is read too, and its tensor collides with a shard's
    d = tmp_path / "noindex"
    d.mkdir()
    for f in os.listdir(os.path.join(G, "sharded")):
        if f.endswith(".safetensors"):
            (d / f).write_bytes(open(os.path.join(G, "sharded", f), "rb").read())
    with pytest.raises(SystemExit) as e:
        run(str(d))
    assert str(e.value) == "ERROR: tensor 'model.norm.weight' present in multiple shards"
    (d / "consolidated.safetensors").unlink()
    rc, _ = run(str(d), output_dir=str(tmp_path / "o"))
    assert rc == 0
    assert open(tmp_path / "o" / "model.fp16.bin", "rb").read() == \
        open(os.path.join(G, "sharded.bundle", "model.fp16.bin"), "rb").read()
    assert json.load(open(tmp_path / "o" / "model.fp16.meta.json"))["model_id"] == "noindex"


@pytest.mark.parametrize("tag,against", [("mismatch", "single.other.meta.json"),
                                         ("match", os.path.join("single.bundle", "model.fp16.meta.json"))])
def test_check_against_report_is_the_reference_tools(tmp_path, tag, against):
    want = open(os.path.join(G, f"single.check_{tag}.txt")).read()
    want_rc, want_text = int(want.split("\n", 1)[0].split()[1]), want.split("\n", 1)[1]
    rc, text = run(os.path.join(G, "single.safetensors"), check=os.path.join(G, against))
    assert rc == want_rc
    assert text.replace(G + os.sep, "") == want_text
    assert not os.listdir(tmp_path)                                     # nothing written
    # with an output directory a mismatch is reported but the bundle is still written, status 0
    rc, _ = run(os.path.join(G, "single.safetensors"), check=os.path.join(G, against), output_dir=str(tmp_path))
    assert rc == 0 and os.path.exists(tmp_path / "model.fp16.bin")


def _st(path, entries, pad=0):
    header, blobs, off = {}, b"", 0
    for name, code, raw, shape in entries:
        header[name] = {"dtype": code, "shape": shape, "data_offsets": [off, off + len(raw)]}
        blobs += raw
        off += len(raw)
    text = json.dumps(header).encode() + b" " * pad
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)) + text + blobs)


def test_every_bf16_pattern_converts_like_fp32_then_round_to_nearest_even(tmp_path):
    # all 65 536 bf16 encodings: the value is the fp32 with those upper 16 bits, exactly
    bits = np.arange(65536, dtype="<u2")
    _st(tmp_path / "a.safetensors", [("all", "BF16", bits.tobytes(), [65536])], pad=5)
    rc, _ = run(str(tmp_path / "a.safetensors"), output_dir=str(tmp_path / "o"))
    assert rc == 0
    got = np.fromfile(tmp_path / "o" / "model.fp16.bin", dtype=np.uint16)
    f32 = (bits.astype(np.uint32) << 16).view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = f32.astype(np.float64).astype(np.float16).view(np.uint16)   # double -> half is a single rounding
    nan = np.isnan(f32)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float16)))


def test_integer_and_f64_inputs_round_once(tmp_path):
    i64 = np.array([2049, 2051, -2049, 65519, 65520, 4097, 1 << 40], "<i8")          # ties and overflow
    f64 = np.array([1.0 + 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -30, 65519.999, 5.9604644775390625e-08 / 2], "<f8")
    _st(tmp_path / "a.safetensors", [("i", "I64", i64.tobytes(), [7]), ("f", "F64", f64.tobytes(), [2, 2])])
    rc, _ = run(str(tmp_path / "a.safetensors"), output_dir=str(tmp_path / "o"))
    got = np.fromfile(tmp_path / "o" / "model.fp16.bin", dtype=np.float16)
    # sorted order: "f" first.  1 + 2^-11 is a tie -> even (1.0); a hair above it rounds up
    assert list(got[:4].astype(np.float64)) == [1.0, 1.0 + 2.0 ** -10, 65504.0, 0.0]
    assert list(got[4:].astype(np.float64)) == [2048.0, 2052.0, -2048.0, 65504.0, np.inf, 4096.0, np.inf]


def test_errors_are_the_reference_tools(tmp_path):
    with pytest.raises(SystemExit) as e:
        run(str(tmp_path / "missing"))
    assert str(e.value) == f"ERROR: --input not found: {tmp_path / 'missing'}"
    (tmp_path / "x.bin").write_bytes(b"")
    with pytest.raises(SystemExit) as e:
        run(str(tmp_path / "x.bin"))
    assert str(e.value) == f"ERROR: {tmp_path / 'x.bin'} is not a .safetensors file"
    (tmp_path / "empty").mkdir()
    with pytest.raises(SystemExit) as e:
        run(str(tmp_path / "empty"))
    assert str(e.value) == f"ERROR: no .safetensors found under {tmp_path / 'empty'}"
    _st(tmp_path / "bad.safetensors", [("t", "F8_E4M3", b"\0" * 4, [4])])
    with pytest.raises(SystemExit) as e:
        run(str(tmp_path / "bad.safetensors"))
    assert str(e.value) == "ERROR: t: unsupported dtype F8_E4M3"
    _st(tmp_path / "short.safetensors", [("t", "F32", b"\0" * 12, [4])])
    with pytest.raises(SystemExit) as e:
        run(str(tmp_path / "short.safetensors"))
    assert str(e.value) == "ERROR: t: element count 3 != prod(shape) 4"


def test_command_line_and_the_quantiser_behind_it(tmp_path):
    # the tool's output is what the bundle quantiser and the library's loader take as input
    tool = os.path.join(ROOT, "adreno-llms_amd", "convert_hf_to_bin.py")
    r = subprocess.run([sys.executable, tool, "--input", os.path.join(G, "sharded"), "--output-dir", str(tmp_path)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert r.stdout.splitlines()[-1] == f"Wrote {tmp_path / 'model.fp16.meta.json'} ✓"
    r = subprocess.run([sys.executable, tool, "--hf-repo-id", "some/model"], capture_output=True, text=True)
    assert r.returncode == 1 and r.stderr.startswith("ERROR:")
    bt = importlib.import_module("adreno-llms_amd.bundle_tools")
    meta = bt.quantize_bundle("int8", str(tmp_path / "model.fp16.bin"), str(tmp_path / "model.fp16.meta.json"),
                              str(tmp_path / "q.bin"), str(tmp_path / "q.json"), suffixes=(".w",))
    assert meta["tensors"]["model.layers.0.w"]["dtype"] == "int8"
    assert "model.layers.0.w.scale" in meta["tensors"]
