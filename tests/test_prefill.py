"""A prompt at once (mi_decoder_prefill: Model::forward with seq_len = M, QW/src/model.cpp:243-376,
every projection an M-row call).

The reference's quantised prefill is a loop of single-token steps (LF/src/model.cpp:243-250), so the
expected result of a prompt is what the CPU harness (oracle/decode.c) leaves after feeding the
tokens one by one: with the M > 1 projections as rows of GEMV (mi_set_gemm_mode(1)) the logits
after the prompt and after further single-token steps (which read the cache rows the prompt
wrote) must equal the harness's bit for bit; on the matrix cores the sums run in another order
and the logits are compared within a tolerance stated in the test."""
import numpy as np
import pytest

from decode_harness import PROMPT, QWEN25_05B, SMOL, TINY, GpuDecoder, KindModel, Model, greedy
from helpers import mil


def _f32(bits):
    return bits.view(np.float16).astype(np.float32)


def _prompt(n, vocab, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, n)]


def _oracle(m, prompt, n_new, **kw):
    vocab = m.cfg["vocab"]
    logits = np.empty(vocab, np.uint16)
    toks, margins = greedy(m, prompt, n_new, last_logits=logits, **kw)
    return toks, margins, logits


@pytest.mark.gpu
@pytest.mark.parametrize("name,cfg,kind,n_prompt", [
    ("tiny-int8", TINY, "i8", 6), ("tiny-int8-one-token", TINY, "i8", 1), ("tiny-int8-long", TINY, "i8", 37),
    ("smol-int8", SMOL, "i8", 19), ("smol-fp16", SMOL, "f16", 6), ("smol-q4", SMOL, "q4", 6)])
def test_prompt_as_rows_of_gemv_equals_token_by_token_bit_for_bit(name, cfg, kind, n_prompt):
    assert mil.lib().mi_init(0) == 1
    mil.lib().mi_set_gemm_mode(1)
    mil.lib().mi_set_gemv_mode(0)           # Q4: the same (exact) GEMV in the steps and in the prompt's rows
    try:
        queue = mil.Queue()
        m = Model(cfg, seed=21) if kind == "i8" else KindModel(cfg, kind, seed=21)
        cb = None if kind == "i8" else m.oracle_cb()
        prompt = PROMPT if n_prompt == 6 else _prompt(n_prompt, cfg["vocab"], 3)
        prompt = [t % cfg["vocab"] for t in prompt]
        want1, _, logits1 = _oracle(m, prompt, 1, linear_cb=cb)
        want9, _, logits9 = _oracle(m, prompt, 9, linear_cb=cb)
        gd = GpuDecoder(m, queue)
        assert gd.dec.prefill(queue, prompt)
        pos, tok = gd.dec.read(queue)
        assert pos == len(prompt) and [tok] == want1
        assert np.array_equal(gd.logits(), logits1)
        got = [tok]
        for _ in range(8):                   # single-token steps on top of the prompt's cache rows
            assert gd.dec.step(queue)
            got.append(gd.dec.read(queue)[1])
        assert got == want9
        assert np.array_equal(gd.logits(), logits9)
        gd.close()
    finally:
        mil.lib().mi_set_gemm_mode(0)
        mil.lib().mi_set_gemv_mode(1)


@pytest.mark.gpu
def test_prompt_in_two_parts_and_after_steps():
    """A prompt continued at pos0 > 0 (rows below pos0 are read from the cache), a shorter prompt
    after a longer one (the activation rows are reused), and a prompt after single-token steps."""
    assert mil.lib().mi_init(0) == 1
    mil.lib().mi_set_gemm_mode(1)
    try:
        queue = mil.Queue()
        m = Model(TINY, seed=4)
        prompt = _prompt(40, TINY["vocab"], 9)
        want, _, logits = _oracle(m, prompt, 1)
        gd = GpuDecoder(m, queue)
        assert gd.dec.prefill(queue, prompt[:25]) and gd.dec.prefill(queue, prompt[25:], 25)
        assert gd.dec.read(queue) == (40, want[0])
        assert np.array_equal(gd.logits(), logits)
        # steps for the first 10 tokens, the rest as a prompt
        assert gd.dec.reset(queue, 0, prompt[0])
        for t in prompt[1:10]:
            assert gd.dec.step(queue) and gd.dec.set_token(queue, t)
        assert gd.dec.step(queue)                         # consumes prompt[9]
        assert gd.dec.prefill(queue, prompt[10:], 10)
        assert gd.dec.read(queue) == (40, want[0])
        assert np.array_equal(gd.logits(), logits)
        # refused: beyond the cache, empty
        assert not gd.dec.prefill(queue, prompt, TINY["max_pos"] - 39)
        assert not gd.dec.prefill(queue, [], 0)
        assert gd.dec.read(queue) == (40, want[0])        # a refused call changes nothing
        gd.close()
    finally:
        mil.lib().mi_set_gemm_mode(0)


@pytest.mark.gpu
def test_reserved_prompt_room_means_no_allocation_in_prefill():
    """After mi_decoder_reserve_prompt the prompts that fit allocate nothing (the device's free memory
    does not move across them) and give the results of a decoder that made its room on the way."""
    import ctypes
    assert mil.lib().mi_init(0) == 1
    hip = ctypes.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    mil.lib().mi_set_gemm_mode(1)
    try:
        queue = mil.Queue()
        m = Model(SMOL, seed=6)
        prompt = _prompt(40, SMOL["vocab"], 11)
        want, _, logits = _oracle(m, prompt, 1)
        gd = GpuDecoder(m, queue)
        assert not gd.dec.reserve_prompt(queue, 0) and not gd.dec.reserve_prompt(queue, SMOL["max_pos"] + 1)
        assert gd.dec.reserve_prompt(queue, 40)
        before = free_bytes()
        assert gd.dec.prefill(queue, prompt[:17]) and gd.dec.prefill(queue, prompt[17:], 17)
        assert gd.dec.prefill(queue, prompt)
        queue.finish()
        assert free_bytes() == before
        assert gd.dec.read(queue) == (40, want[0])
        assert np.array_equal(gd.logits(), logits)
        assert gd.dec.reserve_prompt(queue, 12)            # less than there is: nothing to do
        assert free_bytes() == before
        gd.close()
    finally:
        mil.lib().mi_set_gemm_mode(0)


@pytest.mark.gpu
@pytest.mark.parametrize("name,cfg,n_prompt", [("smol", SMOL, 40), ("tiny", TINY, 33), ("smol-f16", SMOL, 40),
                                               ("smol-q4", SMOL, 40)])
def test_prompt_on_the_matrix_cores_within_tolerance(name, cfg, n_prompt):
    """Default mode: the M-row projections run as MFMA GEMMs where the library's estimate favours
    them.  Each projection is within one fp16 step of the rows of GEMV; through the layers of the
    model the logits stay within max-abs 1e-2 of the largest logit and cosine >= 0.9999 of the
    token-by-token ones, and the greedy token is the same wherever the harness's top-1/top-2
    margin exceeds twice the largest difference."""
    assert mil.lib().mi_init(0) == 1
    queue = mil.Queue()
    kind = name.split("-")[1] if "-" in name else "i8"
    m = Model(cfg, seed=33) if kind == "i8" else KindModel(cfg, kind, seed=33)
    prompt = _prompt(n_prompt, cfg["vocab"], 5)
    want, margins, logits = _oracle(m, prompt, 1, linear_cb=None if kind == "i8" else m.oracle_cb())
    gd = GpuDecoder(m, queue)
    assert gd.dec.prefill(queue, prompt)
    pos, tok = gd.dec.read(queue)
    got = _f32(gd.logits())
    gd.close()
    ref = _f32(logits)
    diff = float(np.max(np.abs(got - ref)))
    cos = float(np.dot(got, ref) / (np.linalg.norm(got) * np.linalg.norm(ref)))
    print(f"{name}: max |diff| {diff:.3e} of max |logit| {np.max(np.abs(ref)):.3f}, cosine {cos:.7f}, "
          f"margin {margins[0]:.4f}", flush=True)
    assert pos == n_prompt
    assert diff <= 1e-2 * float(np.max(np.abs(ref))) and cos >= 0.9999
    if margins[0] > 2 * diff:
        assert tok == want[0]


@pytest.mark.gpu
def test_qwen_shaped_prompt_against_single_token_steps_on_device():
    """Qwen2.5-0.5B shapes (24 layers, vocabulary 151 936, int8 per row), a prompt of 48 tokens:
    as rows of GEMV the prompt leaves the logits of 48 single-token steps on the device bit for bit
    (those steps equal the CPU harness in test_decode_tokens.py); on the matrix cores within the
    tolerance above.  Four more tokens decoded from either cache agree in the exact mode."""
    assert mil.lib().mi_init(0) == 1
    queue = mil.Queue()
    m = Model(QWEN25_05B, seed=2024)
    prompt = _prompt(48, QWEN25_05B["vocab"], 12)
    gd = GpuDecoder(m, queue)
    try:
        toks = gd.greedy(prompt, 1)                      # token by token, tokens forced
        step_logits = gd.logits()
        more = [gd.dec.read(queue)[1]]
        for _ in range(4):
            assert gd.dec.step(queue)
            more.append(gd.dec.read(queue)[1])
        mil.lib().mi_set_gemm_mode(1)
        assert gd.dec.prefill(queue, prompt)
        assert gd.dec.read(queue) == (48, toks[0])
        assert np.array_equal(gd.logits(), step_logits)
        again = [toks[0]]
        for _ in range(4):
            assert gd.dec.step(queue)
            again.append(gd.dec.read(queue)[1])
        assert again == more
        mil.lib().mi_set_gemm_mode(0)
        assert gd.dec.prefill(queue, prompt)
        got, ref = _f32(gd.logits()), _f32(step_logits)
        diff = float(np.max(np.abs(got - ref)))
        cos = float(np.dot(got, ref) / (np.linalg.norm(got) * np.linalg.norm(ref)))
        print(f"qwen shapes, 48 tokens on the matrix cores: max |diff| {diff:.3e} of max |logit| "
              f"{np.max(np.abs(ref)):.3f}, cosine {cos:.7f}", flush=True)
        assert diff <= 1e-2 * float(np.max(np.abs(ref))) and cos >= 0.9999
    finally:
        mil.lib().mi_set_gemm_mode(0)
        gd.close()


@pytest.mark.gpu
@pytest.mark.parametrize("name,cfg,n_prompt", [
    # head_dim 128, four query heads per key/value head, three tiles of 64 cache rows, the cache filled to its last row
    ("wide_heads", dict(hidden=1024, inter=1536, n_heads=8, n_kv_heads=2, head_dim=128, n_layers=2, vocab=2048,
                        max_pos=150, rms_eps=1e-6, rope_theta=500000.0), 141),
    # nine query heads per key/value head: more than a block of the grouped kernel serves, one block per head and row
    ("nine_per_group", dict(hidden=576, inter=1536, n_heads=9, n_kv_heads=1, head_dim=64, n_layers=1, vocab=1024,
                            max_pos=80, rms_eps=1e-5, rope_theta=100000.0), 71),
    # a head width that is no whole number of wavefronts: the per-head kernels on both sides
    ("head_dim_80", dict(hidden=640, inter=1024, n_heads=8, n_kv_heads=2, head_dim=80, n_layers=2, vocab=1024,
                         max_pos=100, rms_eps=1e-6, rope_theta=10000.0), 75),
    # eight heads per group over 1800 positions: 66 KB of scores per block, beyond the 64 KB a kernel gets
    # unasked; checked against the device's own single-token steps (the CPU harness would need 15 s)
    ("long_context", dict(hidden=512, inter=512, n_heads=8, n_kv_heads=1, head_dim=64, n_layers=1, vocab=512,
                          max_pos=1800, rms_eps=1e-6, rope_theta=1000000.0), 1800),
])
def test_prompt_other_geometries_bit_for_bit(name, cfg, n_prompt):
    assert mil.lib().mi_init(0) == 1
    mil.lib().mi_set_gemm_mode(1)
    try:
        queue = mil.Queue()
        m = Model(cfg, seed=17)
        prompt = _prompt(n_prompt, cfg["vocab"], 8)
        gd = GpuDecoder(m, queue)
        if name == "long_context":
            want = gd.greedy(prompt, 1)
            logits = gd.logits()
        else:
            want, _, logits = _oracle(m, prompt, 1)
        assert gd.dec.prefill(queue, prompt)
        assert gd.dec.read(queue) == (n_prompt, want[0])
        assert np.array_equal(gd.logits(), logits)
        gd.close()
    finally:
        mil.lib().mi_set_gemm_mode(0)
