"""Greedy token IDs over 32 steps on seeded random-init weights (config 4).

The same CPU harness (oracle/decode.c) runs twice: with the oracle's int8 GEMV behind
every projection, and with the GPU library behind every projection.  Token lists must be
identical; since the GEMV kernels are bit-exact, so are the logits."""
import numpy as np
import pytest

import oracle_lib as O
from decode_harness import PROMPT, QWEN25_05B, TINY, GpuDecoder, GpuLinear, Model, greedy
from helpers import mil


def test_harness_is_deterministic_and_callback_equals_builtin():
    m = Model(TINY, seed=7)
    toks, margins = greedy(m, PROMPT, 12)
    toks2, _ = greedy(m, PROMPT, 12, threads=1)
    assert toks == toks2 and len(toks) == 12
    assert all(0 <= t < TINY["vocab"] for t in toks)

    def cb(idx, x_ptr, y_ptr):                      # the oracle GEMV, reached through the callback
        N, K = m.shapes[idx]
        x = np.ctypeslib.as_array((np.ctypeslib.ctypes.c_uint16 * K).from_address(x_ptr))
        y = np.ctypeslib.as_array((np.ctypeslib.ctypes.c_uint16 * N).from_address(y_ptr))
        y[:] = O.gemv_i8(x.view(np.float16), m.w8[idx], m.ws[idx].view(np.uint16))

    toks3, _ = greedy(m, PROMPT, 12, linear_cb=cb)
    assert toks3 == toks
    # a different model gives a different continuation (the check is not vacuous)
    assert greedy(Model(TINY, seed=8), PROMPT, 12)[0] != toks


@pytest.mark.gpu
def test_tiny_model_tokens_identical_on_gpu():
    assert mil.lib().mi_init(0) == 1
    queue = mil.Queue()
    m = Model(TINY, seed=11)
    want, _ = greedy(m, PROMPT, 32)
    gl = GpuLinear(m, queue)
    got, _ = greedy(m, PROMPT, 32, linear_cb=gl)
    gl.close()
    assert got == want
    assert gl.calls == (len(PROMPT) + 32) * (TINY["n_layers"] * 7 + 1)


@pytest.mark.gpu
def test_qwen_shaped_32_greedy_tokens_identical_on_gpu():
    """Qwen2.5-0.5B shapes: 24 x {q 896x896, k/v 128x896, o 896x896, gate/up 4864x896,
    down 896x4864} + lm_head 151936x896, int8 per row, prompt of 6 ids, 32 greedy steps."""
    assert mil.lib().mi_init(0) == 1
    queue = mil.Queue()
    print("building the model", flush=True)
    m = Model(QWEN25_05B, seed=2024)
    print("oracle run", flush=True)
    want, margins = greedy(m, PROMPT, 32)
    print("gpu run", flush=True)
    gl = GpuLinear(m, queue)
    got, _ = greedy(m, PROMPT, 32, linear_cb=gl)
    gl.close()
    print("tokens", got, "min top-1/top-2 margin", min(margins), flush=True)
    assert got == want
    assert len(set(got)) > 1


@pytest.mark.gpu
@pytest.mark.parametrize("graph", [False, True], ids=["stream", "graph"])
def test_tiny_model_whole_step_on_device(graph):
    """mi_decoder_*: every kernel of the step on the GPU, tokens chained in device memory; the token
    list equals the CPU harness's (the small kernels repeat its operations in its order)."""
    assert mil.lib().mi_init(0) == 1
    mil.lib().mi_set_gemv_mode(0)
    try:
        queue = mil.Queue()
        m = Model(TINY, seed=11)
        want, _ = greedy(m, PROMPT, 32)
        gd = GpuDecoder(m, queue)
        got = gd.greedy(PROMPT, 32, graph=graph)
        gd.close()
        assert got == want
    finally:
        mil.lib().mi_set_gemv_mode(1)


@pytest.mark.gpu
def test_qwen_shaped_whole_step_on_device_graph_replay():
    assert mil.lib().mi_init(0) == 1
    queue = mil.Queue()
    m = Model(QWEN25_05B, seed=2024)
    want, _ = greedy(m, PROMPT, 32)
    gd = GpuDecoder(m, queue)
    got = gd.greedy(PROMPT, 32, graph=True)
    pos, _ = gd.dec.read(queue)
    gd.close()
    print("tokens", got, flush=True)
    assert got == want
    assert pos == len(PROMPT) - 1 + 32       # the first prompt token is set by reset, every later token costs a step
