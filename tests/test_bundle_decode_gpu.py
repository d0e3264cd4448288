"""From a bundle on disk to greedy tokens: the path a port of the reference takes at start-up and per token.

An fp16 bundle in the reference's layout (scripts/convert_hf_to_bin.py:149-170) with a Qwen2-shaped model's
tensors under their Hugging Face names is quantised to an int8 and to a Q4 bundle by this package's writer
(byte-identical to LF/scripts/quantize_weights.py / quantize_q4.py, tests/test_bundle_tools.py), loaded with
Weights::load / get_buffer and the NNOPT_QUANT registration loop (QW/src/weights.cpp:165-293,
LF/src/main.cpp:527-566: mi_bundle_open / _upload / _device_ptr), and the decoder is built on the device
pointers the bundle hands out.  32 greedy tokens and every bit of the last step's logits must equal the CPU
harness's run on the same bytes (Model::forward_greedy, QW/src/model.cpp:387-500)."""
import importlib
import json

import numpy as np
import pytest

import oracle_lib as O
from decode_harness import PROMPT, SMOL, TINY, KindModel, Model, greedy
from helpers import mil

bt = importlib.import_module("adreno-llms_amd.bundle_tools")
pytestmark = pytest.mark.gpu

PROJ = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
        "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")
SUFFIXES = tuple(p.split(".")[1] + ".weight" for p in PROJ) + ("lm_head.weight",)


def _fp16_tensors(model, seed):
    """The fp16 tensors the harness's model was quantised from, under Hugging Face names."""
    c, s = model.cfg, seed * 1000
    t = {"model.embed_tokens.weight": model.embed, "model.norm.weight": model.final_norm}
    for l in range(c["n_layers"]):
        pre = f"model.layers.{l}."
        for j, p in enumerate(PROJ):
            N, K = model.shapes[l * 7 + j]
            t[pre + p + ".weight"] = mil.synth_normal_f16(s + 1 + l * 7 + j, 0.02, (N, K))
        t[pre + "self_attn.q_proj.bias"] = model.bq[l]
        t[pre + "self_attn.k_proj.bias"] = model.bk[l]
        t[pre + "self_attn.v_proj.bias"] = model.bv[l]
        t[pre + "input_layernorm.weight"] = model.in_norm[l]
        t[pre + "post_attention_layernorm.weight"] = model.post_norm[l]
    t["lm_head.weight"] = mil.synth_normal_f16(s + 400, 0.02, model.shapes[-1])
    return t


@pytest.mark.parametrize("scheme,cfg", [("int8", TINY), ("q4", TINY), ("int8", SMOL)], ids=["int8-tiny", "q4-tiny", "int8-smol"])
def test_greedy_tokens_from_a_bundle_on_disk(tmp_path, scheme, cfg):
    assert mil.lib().mi_init(0) == 1
    seed = 17
    model = Model(cfg, seed=seed) if scheme == "int8" else KindModel(cfg, "q4", seed=seed)
    fp16 = (str(tmp_path / "model.fp16.bin"), str(tmp_path / "model.fp16.meta.json"))
    bt.write_fp16_bundle(_fp16_tensors(model, seed), *fp16, model_id="synthetic/qwen2-shaped")
    qbin, qmeta = str(tmp_path / f"model.{scheme}.bin"), str(tmp_path / f"model.{scheme}.meta.json")
    bt.quantize_bundle(scheme, *fp16, qbin, qmeta, suffixes=SUFFIXES)
    meta = json.load(open(qmeta))

    w = mil.Weights()
    assert w.load(qbin, qmeta)
    names = [f"model.layers.{l}.{p}.weight" for l in range(cfg["n_layers"]) for p in PROJ] + ["lm_head.weight"]
    # the file holds what the harness's model holds: same quantiser, same bytes
    for i, name in enumerate(names):
        assert meta["tensors"][name]["dtype"] == ("int8" if scheme == "int8" else "q4_packed"), name
        if scheme == "int8":
            assert np.array_equal(w.get_host(name), model.w8[i]), name
            assert np.array_equal(w.get_host(name + ".scale"), model.ws[i]), name
        else:
            assert np.array_equal(w.get_host(name), model.wq4[i][0]), name
            assert np.array_equal(w.get_host(name + ".scale"), model.wq4[i][1]), name
    want_logits = np.empty(cfg["vocab"], np.uint16)
    want, _ = greedy(model, PROMPT, 32, linear_cb=model.oracle_cb() if scheme == "q4" else None, last_logits=want_logits)

    print(f"bundle -> device -> decoder, {scheme}, hidden {cfg['hidden']}", flush=True)
    assert w.upload() == len(names)
    L = cfg["n_layers"]
    layer = lambda suffix: [w.get_buffer(f"model.layers.{l}.{suffix}") for l in range(L)]
    bufs = dict(embed=w.get_buffer("model.embed_tokens.weight"), final_norm=w.get_buffer("model.norm.weight"),
                lm_head=w.get_buffer("lm_head.weight"),
                in_norm=layer("input_layernorm.weight"), post_norm=layer("post_attention_layernorm.weight"),
                bq=layer("self_attn.q_proj.bias"), bk=layer("self_attn.k_proj.bias"), bv=layer("self_attn.v_proj.bias"),
                wq=layer("self_attn.q_proj.weight"), wk=layer("self_attn.k_proj.weight"), wv=layer("self_attn.v_proj.weight"),
                wo=layer("self_attn.o_proj.weight"), wgate=layer("mlp.gate_proj.weight"), wup=layer("mlp.up_proj.weight"),
                wdown=layer("mlp.down_proj.weight"))
    assert all(bufs[k] for k in ("embed", "final_norm", "lm_head")) and all(all(v) for k, v in bufs.items() if isinstance(v, list))
    mil.lib().mi_set_gemv_mode(0)                       # the reference's order of operations: bit for bit
    queue = mil.Queue()
    try:
        dec = mil.Decoder(cfg, bufs)
        vocab = cfg["vocab"]
        assert dec.reset(queue, 0, PROMPT[0] % vocab) and dec.step(queue)      # first use of the kernels, outside the recording
        queue.finish()
        assert dec.reset(queue, 0, PROMPT[0] % vocab)
        with mil.Graph(queue) as g:
            assert dec.step(queue)
        for t in PROMPT[1:]:
            g.launch()
            assert dec.set_token(queue, t % vocab)
        got = []
        for _ in range(32):
            g.launch()
            got.append(dec.read(queue)[1])
        got_logits = np.empty(vocab, np.uint16)
        queue.finish()
        assert mil.lib().mi_memcpy_d2h(got_logits.ctypes.data, dec.logits_ptr, vocab * 2, queue.handle)
        dec.close()
    finally:
        mil.lib().mi_set_gemv_mode(1)
    print("tokens", got, flush=True)
    assert got == want and len(set(got)) > 1
    assert np.array_equal(got_logits, want_logits)
    w.close()
