"""Bundle writers (adreno-llms_amd/bundle_tools.py) against files the reference's own scripts wrote
from the same tiny fp16 bundle (tests/golden/bundle/, made by tests/golden/make_bundle_vectors.py),
and against the library's bundle reader."""
import importlib
import json
import os

import numpy as np
import pytest

from helpers import mil

bt = importlib.import_module("adreno-llms_amd.bundle_tools")
G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "bundle")
FP16 = (os.path.join(G, "tiny.fp16.bin"), os.path.join(G, "tiny.fp16.meta.json"))

VARIANTS = [
    ("int8", "int8", {}),
    ("int8_embed_alias", "int8", {"quantize_embed": True, "emit_lm_head": True}),
    ("q4", "q4", {}),
    ("q4_alias", "q4", {"emit_lm_head": True}),
]


@pytest.mark.parametrize("tag,scheme,opts", VARIANTS, ids=[v[0] for v in VARIANTS])
def test_quantised_bundle_is_byte_identical_to_the_reference_tools_output(tmp_path, tag, scheme, opts):
    want_bin = open(os.path.join(G, f"tiny.{tag}.bin"), "rb").read()
    want_meta_text = open(os.path.join(G, f"tiny.{tag}.meta.json")).read()
    want_meta = json.loads(want_meta_text)
    out_bin, out_meta = str(tmp_path / "o.bin"), str(tmp_path / "o.meta.json")
    # the free-text "method" note is the reference author's wording; everything else must come out of the tool
    got = bt.quantize_bundle(scheme, *FP16, out_bin, out_meta, method=want_meta["quantization"]["method"], **opts)
    assert open(out_bin, "rb").read() == want_bin
    assert got == want_meta
    assert open(out_meta).read() == want_meta_text
    # defaults differ from the reference only in that note
    got2 = bt.quantize_bundle(scheme, *FP16, out_bin, out_meta, **opts)
    got2["quantization"]["method"] = want_meta["quantization"]["method"]
    assert got2 == want_meta


def test_fp16_writer_layout(tmp_path):
    rng = np.random.default_rng(3)
    tensors = {"b.weight": rng.standard_normal((3, 8)).astype(np.float16),
               "a.weight": rng.standard_normal((5,)).astype(np.float32),      # cast to fp16
               "c.k": rng.standard_normal((2, 1, 3)).astype(np.float16)}
    meta = bt.write_fp16_bundle(tensors, str(tmp_path / "m.bin"), str(tmp_path / "m.json"), model_id="x/y")
    assert list(meta["tensors"]) == ["a.weight", "b.weight", "c.k"]            # sorted, and in that order in the file
    off = 0
    raw = open(tmp_path / "m.bin", "rb").read()
    for name in ["a.weight", "b.weight", "c.k"]:
        t = meta["tensors"][name]
        a = np.asarray(tensors[name]).astype(np.float16)
        assert t == {"offset": off, "shape": list(a.shape), "dtype": "float16", "num_elements": a.size,
                     "size_bytes": a.nbytes}
        assert raw[off:off + a.nbytes] == a.tobytes()
        off += a.nbytes
    assert meta["total_bytes"] == off == len(raw)
    assert json.load(open(tmp_path / "m.json")) == meta


@pytest.mark.parametrize("scheme", ["int8", "q4"])
def test_written_bundle_reads_back_through_the_library(tmp_path, scheme):
    out_bin, out_meta = str(tmp_path / "o.bin"), str(tmp_path / "o.meta.json")
    meta = bt.quantize_bundle(scheme, *FP16, out_bin, out_meta, emit_lm_head=True)
    w = mil.Weights()
    assert w.load(out_bin, out_meta)
    assert sorted(w.all_keys()) == sorted(meta["tensors"])
    src = mil.Weights()
    assert src.load(*FP16)
    name = "model.layers.0.feed_forward.w2.weight"
    fp = src.get_host(name).reshape(64, 96)
    if scheme == "int8":
        q, s = mil.quantize_int8(fp)
        assert w.get_dtype(name) == "int8" and w.get_shape(name) == [64, 96]
        assert np.array_equal(w.get_host(name).reshape(64, 96), q)
        assert np.array_equal(w.get_host(name + ".scale").view(np.uint16), s.view(np.uint16))
    else:
        p, s = mil.quantize_q4(fp)
        assert w.get_dtype(name) == "q4_packed" and w.get_shape(name) == [64, 48]
        assert np.array_equal(w.get_host(name).reshape(64, 48), p)
        assert np.array_equal(w.get_host(name + ".scale").view(np.uint16).reshape(64, 3), s.view(np.uint16))
    assert w.get_shape("lm_head.weight") == ([40, 64] if scheme == "int8" else [40, 32])
    assert w.get_dtype("model.embed_tokens.weight") == "float16"
    # pass-through tensors are the input bytes
    assert np.array_equal(w.get_host("model.layers.0.conv.conv.weight").view(np.uint16),
                          src.get_host("model.layers.0.conv.conv.weight").view(np.uint16))


def test_q4_refuses_rows_that_are_not_whole_blocks(tmp_path):
    bt.write_fp16_bundle({"l.feed_forward.w1.weight": np.zeros((4, 48), np.float16)}, str(tmp_path / "a.bin"),
                         str(tmp_path / "a.json"))
    with pytest.raises(RuntimeError, match="not divisible by 32"):
        bt.quantize_bundle("q4", str(tmp_path / "a.bin"), str(tmp_path / "a.json"), str(tmp_path / "b.bin"),
                           str(tmp_path / "b.json"))


def test_command_line(tmp_path):
    rc = bt.main(["int8", "--fp16-bin", FP16[0], "--fp16-meta", FP16[1], "--out-bin", str(tmp_path / "c.bin"),
                  "--out-meta", str(tmp_path / "c.json"), "--suffix", ".self_attn.q_proj.weight"])
    assert rc == 0
    meta = json.load(open(tmp_path / "c.json"))
    kinds = {n: t["dtype"] for n, t in meta["tensors"].items()}
    assert kinds["model.layers.1.self_attn.q_proj.weight"] == "int8"
    assert kinds["model.layers.1.self_attn.k_proj.weight"] == "float16"
