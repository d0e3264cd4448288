"""Host-side tools of the shipped library (quantizers, codec, generator, bundle
reader) against the oracle, the reference's golden vectors and closed forms."""
import json
import os

import numpy as np
import pytest

import oracle_lib as O
from helpers import mil, synth_w

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "quantizer_vectors.npz"))


@pytest.mark.parametrize("K", [64, 896])
def test_quantizers_match_reference_vectors(K):
    q, s = mil.quantize_int8(GOLD[f"int8_w_k{K}"].view(np.float16))
    assert np.array_equal(q, GOLD[f"int8_q_k{K}"])
    assert np.array_equal(s.view(np.uint16), GOLD[f"int8_s_k{K}"])
    p, sc = mil.quantize_q4(GOLD[f"q4_w_k{K}"].view(np.float16))
    assert np.array_equal(p, GOLD[f"q4_p_k{K}"])
    assert np.array_equal(sc.view(np.uint16), GOLD[f"q4_s_k{K}"])


def test_quantizers_match_oracle_on_bulk_data():
    w = synth_w(7, 1000, 896)
    w[17] = 0
    q, s = mil.quantize_int8(w)
    q2, s2 = O.quantize_int8(w)
    assert np.array_equal(q, q2) and np.array_equal(s.view(np.uint16), s2)
    p, sc = mil.quantize_q4(w)
    p2, sc2 = O.quantize_q4(w)
    assert np.array_equal(p, p2) and np.array_equal(sc.view(np.uint16), sc2)


def test_q4_rejects_ragged_k():
    with pytest.raises(RuntimeError):
        mil.quantize_q4(np.zeros((2, 48), np.float16))


def test_codec_matches_numpy():
    L = mil.lib()
    bits = np.arange(0, 65536, 7, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.mi_f16_to_f32(int(b)) for b in bits], np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    rng = np.random.default_rng(5)
    f = (rng.standard_normal(50000) * 10.0 ** rng.uniform(-9, 5, 50000)).astype(np.float32)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([L.mi_f32_to_f16(float(v)) for v in f], np.uint16)
    assert np.array_equal(got, want)


def test_generator_is_seeded_sliceable_and_normal():
    a = mil.synth_normal_f16(42, 0.02, (300000,))
    b = mil.synth_normal_f16(42, 0.02, (300000,))
    c = mil.synth_normal_f16(43, 0.02, (300000,))
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert np.array_equal(mil.synth_normal_f16(42, 0.02, (1000,)), a[:1000])   # prefix-stable
    af = a.astype(np.float64)
    assert abs(af.mean()) < 2e-4 and abs(af.std() - 0.02) < 2e-4
    x = mil.synth_normal_f16(1, 1.0, (200000,)).astype(np.float64)
    assert abs(np.mean(x ** 4) - 3.0) < 0.1                                     # normal kurtosis


def _write_bundle(tmp_path, tensors, extra=None):
    """tensors: name -> (ndarray, dtype string); written in sorted-name order, no padding."""
    meta, chunks, off = {}, [], 0
    for name in sorted(tensors):
        arr, dtype = tensors[name]
        raw = np.ascontiguousarray(arr).tobytes()
        meta[name] = {"offset": off, "shape": list(arr.shape), "dtype": dtype,
                      "num_elements": int(arr.size), "size_bytes": len(raw)}
        chunks.append(raw)
        off += len(raw)
    doc = {"model_id": "synthetic/tiny", "format": "binary", "layout": "row_major", "dtype": "mixed",
           "quantization": {"enabled": True, "bits": 8, "method": "per-row symmetric int8 \"test\""},
           "total_bytes": off, "tensors": meta}
    if extra:
        doc.update(extra)
    bin_path, meta_path = tmp_path / "model.int8.bin", tmp_path / "model.int8.meta.json"
    bin_path.write_bytes(b"".join(chunks))
    meta_path.write_text(json.dumps(doc, indent=2))
    return str(bin_path), str(meta_path)


def test_bundle_reader_layout(tmp_path):
    w = synth_w(3, 12, 64)
    q, s = mil.quantize_int8(w)
    p, sc = mil.quantize_q4(w)
    norm = np.ones(64, np.float16)
    tensors = {
        "model.layers.0.mlp.up_proj.weight": (q, "int8"),
        "model.layers.0.mlp.up_proj.weight.scale": (s, "float16"),
        "model.layers.0.mlp.down_proj.weight": (p, "q4_packed"),
        "model.layers.0.mlp.down_proj.weight.scale": (sc, "float16"),
        "model.norm.weight": (norm, "float16"),
        "model.embed_tokens.weight": (w, "float16"),
    }
    bin_path, meta_path = _write_bundle(tmp_path, tensors)
    W = mil.Weights()
    assert W.load(bin_path, meta_path)
    assert W.all_keys() == sorted(tensors)
    assert W.get_dtype("model.layers.0.mlp.up_proj.weight") == "int8"
    assert W.get_shape("model.layers.0.mlp.down_proj.weight") == [12, 32]      # packed bytes, not weights
    assert W.get_shape("model.layers.0.mlp.down_proj.weight.scale") == [12, 2]
    assert W.get_dtype("nope") == "" and not W.has_tensor("nope")
    for name, (arr, _) in tensors.items():
        assert np.array_equal(W.get_host(name), arr), name
    # each quantised tensor is directly followed by its scale in the file
    total = sum(W.get_size_bytes(k) for k in W.all_keys())
    assert total == os.path.getsize(bin_path)
    W.close()


def test_bundle_reader_rejects_bad_meta(tmp_path, capfd):
    w = synth_w(4, 4, 32)
    bin_path, meta_path = _write_bundle(tmp_path, {"a.weight": (w, "float16")})
    doc = json.loads(open(meta_path).read())
    doc["tensors"]["a.weight"]["size_bytes"] += 64                      # runs past the file
    open(meta_path, "w").write(json.dumps(doc))
    assert not mil.Weights().load(bin_path, meta_path)
    assert "exceeds file bounds" in capfd.readouterr().err
    assert not mil.Weights().load(bin_path, str(tmp_path / "missing.json"))
    assert not mil.Weights().load(str(tmp_path / "missing.bin"), meta_path)
    open(meta_path, "w").write("{ not json")
    assert not mil.Weights().load(bin_path, meta_path)
