"""GPU parity of the GEMV path, through the C ABI, against the CPU oracle.

Bar: bit-exact fp16 outputs (the HIP kernels evaluate the reference kernels' sum in
the same order as the oracle, so even the tolerance of max-abs/rel 1e-3 and cosine
>= 0.9999 that the task states is not needed); unpack / dequant views bit-exact."""
import numpy as np
import pytest

import oracle_lib as O
from helpers import assert_tolerance, mil, synth_w, synth_x

pytestmark = pytest.mark.gpu

# (N, K): the Qwen2.5-0.5B projections, SmolLM2 and LFM2 shapes, ragged N, generic K
SHAPES_I8 = [(1536, 576), (576, 1536), (4864, 896), (896, 4864), (128, 896), (896, 896), (1152, 896),
             (4608, 1024), (1024, 4608), (1024, 2560), (37, 896), (5, 256), (1001, 1024), (3, 4864),
             (64, 320), (13, 36), (7, 4), (2049, 2048), (9, 8200),
             (4100, 4864), (4099, 4608), (8200, 2560), (20001, 1536), (8200, 2048), (8200, 960), (2560, 960)]   # long rows, enough of them for any lane tile
SHAPES_Q4 = [(4864, 896), (896, 4864), (128, 896), (4608, 1024), (1024, 4608), (1024, 2560), (37, 896),
             (5, 256), (3, 32), (64, 320), (11, 96), (1001, 1024), (9, 8192),
             (4100, 4864), (4099, 4608), (8200, 2560), (8200, 2048), (37, 2048), (8200, 960), (2560, 960)]


@pytest.fixture(scope="module")
def queue():
    assert mil.lib().mi_init(0) == 1, "no gfx950 device"
    mil.lib().mi_set_gemv_mode(0)          # reference evaluation order for every kind (bit-exact)
    q = mil.Queue()
    yield q
    q.finish()
    mil.lib().mi_set_gemv_mode(1)


def _run_linear(queue, M, N, K, x, W_host, scale_host=None, kind="f16", canary=True):
    """Upload, register, call pytorch_linear, read back (with guard halves around out)."""
    xb = mil.Buffer.from_host(x)
    Wb = mil.Buffer.from_host(W_host)
    sb = mil.Buffer.from_host(scale_host) if scale_host is not None else None
    if kind == "i8":
        assert mil.nnopt_register_int8_weight(Wb, sb, N, K)
    elif kind == "q4":
        assert mil.nnopt_register_q4_weight(Wb, sb, N, K)
    pad = 64
    guard = np.full(M * N + 2 * pad, 0x7BCD, np.uint16)
    ob = mil.Buffer.from_host(guard)
    assert mil.pytorch_linear(queue, M, N, K, xb, Wb, ob.ptr + 2 * pad)
    queue.finish()
    full = ob.read(np.uint16, guard.shape)
    assert np.all(full[:pad] == 0x7BCD) and np.all(full[-pad:] == 0x7BCD), "wrote outside out[M,N]"
    mil.nnopt_unregister_weight(Wb)
    return full[pad:-pad].reshape(M, N)


@pytest.mark.parametrize("N,K", SHAPES_I8)
def test_int8_gemv_bit_exact(queue, N, K):
    print(f"int8 gemv N={N} K={K}", flush=True)
    W, x = synth_w(100 + N, N, K), synth_x(200 + K, K)
    q, s = mil.quantize_int8(W)
    got = _run_linear(queue, 1, N, K, x, q, s, "i8")[0]
    want = O.gemv_i8(x, q, s.view(np.uint16))
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {N} differ"


@pytest.mark.parametrize("N,K", SHAPES_Q4)
def test_q4_gemv_bit_exact(queue, N, K):
    print(f"q4 gemv N={N} K={K}", flush=True)
    W, x = synth_w(300 + N, N, K), synth_x(400 + K, K)
    p, sc = mil.quantize_q4(W)
    got = _run_linear(queue, 1, N, K, x, p, sc, "q4")[0]
    want = O.gemv_q4(x, p, sc.view(np.uint16))
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {N} differ"


@pytest.mark.parametrize("N,K", SHAPES_I8)
def test_fp16_gemv_bit_exact(queue, N, K):
    print(f"fp16 gemv N={N} K={K}", flush=True)
    W, x = synth_w(500 + N, N, K), synth_x(600 + K, K)
    got = _run_linear(queue, 1, N, K, x, W)[0]
    want = O.gemv_f16(x, W)
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {N} differ"


def test_all_q4_byte_values_and_x_special_values(queue):
    # every packed byte value occurs; x holds subnormals, +-0 and large values
    N, K = 64, 1024
    rng = np.random.default_rng(7)
    p = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    p[0, :256] = np.arange(256, dtype=np.uint8)
    sc = synth_w(8, N, K // 32, 0.01)
    x = synth_x(9, K)
    x[::7] = np.float16(6e-8)          # smallest subnormal
    x[1::7] = np.float16(-3e-6)
    x[2::7] = np.float16(-0.0)
    x[3::97] = np.float16(1000.0)
    got = _run_linear(queue, 1, N, K, x, p, sc, "q4")[0]
    assert np.array_equal(got, O.gemv_q4(x, p, sc.view(np.uint16)))
    q = rng.integers(-127, 128, (N, K)).astype(np.int8)
    q[1, :255] = np.arange(-127, 128, dtype=np.int8)
    s = np.abs(synth_w(10, 1, N, 0.01))[0]
    got = _run_linear(queue, 1, N, K, x, q, s, "i8")[0]
    assert np.array_equal(got, O.gemv_i8(x, q, s.view(np.uint16)))


def test_unit_vectors_return_dequantised_columns(queue):
    N, K = 512, 896
    W = synth_w(11, N, K)
    q, s = mil.quantize_int8(W)
    p, sc = mil.quantize_q4(W)
    nib = np.stack([p & 15, p >> 4], -1).reshape(N, K).astype(np.float32) - 8
    for k in (0, 5, 255, 256, 767, 768, 895):
        x = np.zeros(K, np.float16)
        x[k] = 1.0
        want = (q[:, k].astype(np.float32) * s.astype(np.float32)).astype(np.float16)
        assert np.array_equal(_run_linear(queue, 1, N, K, x, q, s, "i8")[0].view(np.float16), want)
        want = (nib[:, k] * sc[:, k // 32].astype(np.float32)).astype(np.float16)
        assert np.array_equal(_run_linear(queue, 1, N, K, x, p, sc, "q4")[0].view(np.float16), want)
        assert np.array_equal(_run_linear(queue, 1, N, K, x, W)[0].view(np.float16), W[:, k])


def test_dequant_and_unpack_views_bit_exact(queue):
    N, K = 300, 896
    W = synth_w(12, N, K)
    q, s = mil.quantize_int8(W)
    p, _ = mil.quantize_q4(W)
    qb, sb, out = mil.Buffer.from_host(q), mil.Buffer.from_host(s), mil.Buffer(N * K * 2)
    assert mil.dequant_int8_weight_to_fp16(queue, qb, sb, N, K, out)
    queue.finish()
    want = np.empty((N, K), np.uint16)
    O.lib.orc_dequant_int8_to_f16(q, s.view(np.uint16), N, K, want)
    assert np.array_equal(out.read(np.uint16, (N, K)), want)
    pb, out8 = mil.Buffer.from_host(p), mil.Buffer(N * K)
    assert mil.unpack_q4_to_int8(queue, pb, N, K, out8)
    queue.finish()
    want8 = np.empty((N, K), np.int8)
    O.lib.orc_unpack_q4(p, N, K, want8)
    assert np.array_equal(out8.read(np.int8, (N, K)), want8)


@pytest.mark.parametrize("kind", ["i8", "q4", "f16"])
def test_longest_rows(queue, kind, capfd):
    """K = 32 768, the longest row the library takes (x fills 64 KB of LDS), bit for bit; one step more is
    refused with an error line and nothing is written."""
    N, K = 70, 32768
    W, x = synth_w(900, N, K), synth_x(901, K)
    if kind == "i8":
        q, s = mil.quantize_int8(W)
        got, want = _run_linear(queue, 1, N, K, x, q, s, "i8")[0], O.gemv_i8(x, q, s.view(np.uint16))
    elif kind == "q4":
        p, sc = mil.quantize_q4(W)
        got, want = _run_linear(queue, 1, N, K, x, p, sc, "q4")[0], O.gemv_q4(x, p, sc.view(np.uint16))
    else:
        got, want = _run_linear(queue, 1, N, K, x, W)[0], O.gemv_f16(x, W)
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {N} differ"
    K2 = K + 32
    xb, wb, ob = mil.Buffer(K2 * 2), mil.Buffer(4 * K2 * 2), mil.Buffer.from_host(np.full(4, 0x7BCD, np.uint16))
    capfd.readouterr()
    assert not mil.pytorch_linear(queue, 1, 4, K2, xb, wb, ob)
    queue.finish()
    assert "ERROR:" in capfd.readouterr().err
    assert np.all(ob.read(np.uint16, (4,)) == 0x7BCD)


@pytest.mark.parametrize("kind", ["i8", "q4", "f16"])
def test_small_batches_are_rows_of_gemv(queue, kind):
    M, N, K = 5, 1000, 896
    W, X = synth_w(13, N, K), synth_x(14, M, K)
    mil.lib().mi_set_gemm_mode(1)
    try:
        if kind == "i8":
            q, s = mil.quantize_int8(W)
            got = _run_linear(queue, M, N, K, X, q, s, "i8")
            want = O.gemm_i8(X, q, s.view(np.uint16))
        elif kind == "q4":
            p, sc = mil.quantize_q4(W)
            got = _run_linear(queue, M, N, K, X, p, sc, "q4")
            want = O.gemm_q4(X, p, sc.view(np.uint16))
        else:
            got = _run_linear(queue, M, N, K, X, W)
            want = O.gemm_f16(X, W)
    finally:
        mil.lib().mi_set_gemm_mode(0)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("kind", ["i8", "q4", "f16"])
@pytest.mark.parametrize("N,K", [(576, 576), (576, 1536), (896, 4864), (30, 320)])
def test_residual_add_epilogue(queue, kind, N, K):
    if kind == "q4" and K % 32:
        pytest.skip("Q4 needs K % 32 == 0")
    W, x = synth_w(15, N, K), synth_x(16, K)
    res0 = synth_x(17, N)
    xb, rb = mil.Buffer.from_host(x), mil.Buffer.from_host(res0)
    want = res0.view(np.uint16).copy()
    if kind == "i8":
        q, s = mil.quantize_int8(W)
        Wb, sb = mil.Buffer.from_host(q), mil.Buffer.from_host(s)
        assert mil.nnopt_register_int8_weight(Wb, sb, N, K)
        O.lib.orc_gemv_i8_add(O.u16(x), q, s.view(np.uint16), want, N, K)
    elif kind == "q4":
        p, sc = mil.quantize_q4(W)
        Wb, sb = mil.Buffer.from_host(p), mil.Buffer.from_host(sc)
        assert mil.nnopt_register_q4_weight(Wb, sb, N, K)
        O.lib.orc_gemv_q4_add(O.u16(x), p, np.ascontiguousarray(sc.view(np.uint16)), want, N, K)
    else:
        Wb = mil.Buffer.from_host(W)
        O.lib.orc_gemv_f16_add(O.u16(x), O.u16(W), want, N, K)
    assert mil.pytorch_linear_add(queue, 1, N, K, xb, Wb, rb)
    assert not mil.pytorch_linear_add(queue, 2, N, K, xb, Wb, rb)      # M != 1: not taken
    queue.finish()
    assert np.array_equal(rb.read(np.uint16, (N,)), want)
    mil.nnopt_unregister_weight(Wb)


@pytest.mark.parametrize("kind", ["i8", "q4", "f16"])
@pytest.mark.parametrize("N,K", [(4608, 1024), (1536, 576), (4864, 896), (896, 4864), (30, 320)])
def test_silu_gate_epilogue(queue, kind, N, K):
    """pytorch_linear_silu_gate_fused: gate_inout = fp16(silu(gate_inout) * (W3 x)), bit for bit
    against the oracle (LFM2's shape first: K = 1024, N = 4608)."""
    W, x = synth_w(25, N, K), synth_x(26, K)
    gate0 = synth_x(27, N)
    xb, gb = mil.Buffer.from_host(x), mil.Buffer.from_host(gate0)
    want = gate0.view(np.uint16).copy()
    if kind == "i8":
        q, s = mil.quantize_int8(W)
        Wb, sb = mil.Buffer.from_host(q), mil.Buffer.from_host(s)
        assert mil.nnopt_register_int8_weight(Wb, sb, N, K)
        O.lib.orc_gemv_i8_silu_gate(O.u16(x), q, s.view(np.uint16), want, N, K)
    elif kind == "q4":
        p, sc = mil.quantize_q4(W)
        Wb, sb = mil.Buffer.from_host(p), mil.Buffer.from_host(sc)
        assert mil.nnopt_register_q4_weight(Wb, sb, N, K)
        O.lib.orc_gemv_q4_silu_gate(O.u16(x), p, np.ascontiguousarray(sc.view(np.uint16)), want, N, K)
    else:
        Wb = mil.Buffer.from_host(W)
        O.lib.orc_gemv_f16_silu_gate(O.u16(x), O.u16(W), want, N, K)
    assert mil.pytorch_linear_silu_gate_fused(queue, N, K, xb, Wb, gb)
    queue.finish()
    assert np.array_equal(gb.read(np.uint16, (N,)), want)
    mil.nnopt_unregister_weight(Wb)


@pytest.mark.parametrize("kind", ["i8", "f16"])
@pytest.mark.parametrize("N,K", [(1536, 576), (4864, 896), (50, 64), (130, 4104), (2560, 960), (8192, 2048)])
def test_gate_up_silu_epilogue(queue, kind, N, K):
    Wg, Wu, x = synth_w(18, N, K), synth_w(19, N, K), synth_x(20, K)
    xb, ob = mil.Buffer.from_host(x), mil.Buffer(N * 2)
    want = np.empty(N, np.uint16)
    if kind == "i8":
        qg, sg = mil.quantize_int8(Wg)
        qu, su = mil.quantize_int8(Wu)
        gb, ub = mil.Buffer.from_host(qg), mil.Buffer.from_host(qu)
        sgb, sub = mil.Buffer.from_host(sg), mil.Buffer.from_host(su)
        assert mil.nnopt_register_int8_weight(gb, sgb, N, K)
        assert mil.nnopt_register_int8_weight(ub, sub, N, K)
        O.lib.orc_gate_up_silu_i8(O.u16(x), qg, qu, sg.view(np.uint16), su.view(np.uint16), want, N, K)
    else:
        gb, ub = mil.Buffer.from_host(Wg), mil.Buffer.from_host(Wu)
        O.lib.orc_gate_up_silu_f16(O.u16(x), O.u16(Wg), O.u16(Wu), want, N, K)
    assert mil.fused_gate_up_silu_m1(queue, N, K, xb, gb, ub, ob)
    queue.finish()
    got = ob.read(np.uint16, (N,))
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {N} differ"
    mil.nnopt_unregister_weight(gb)
    mil.nnopt_unregister_weight(ub)


def test_dispatch_contract(queue, capfd):
    N, K = 64, 256
    W, x = synth_w(21, N, K), synth_x(22, K)
    q, s = mil.quantize_int8(W)
    xb, qb, sb, ob = mil.Buffer.from_host(x), mil.Buffer.from_host(q), mil.Buffer.from_host(s), mil.Buffer(N * 2)
    # a registered weight called with other dims is refused with an ERROR line
    assert mil.nnopt_register_int8_weight(qb, sb, N, K)
    assert not mil.pytorch_linear(queue, 1, N + 4, K, xb, qb, ob)
    assert "ERROR:" in capfd.readouterr().err
    # null operands and non-positive dims are refused
    assert not mil.pytorch_linear(queue, 1, N, K, None, qb, ob)
    assert not mil.pytorch_linear(queue, 0, N, K, xb, qb, ob)
    # fp16 K that is not a multiple of 4 has no GEMV order in the reference: refused
    Wb = mil.Buffer.from_host(synth_w(23, 8, 6))
    assert not mil.pytorch_linear(queue, 1, 8, 6, xb, Wb, ob)
    capfd.readouterr()
    # an unregistered W is read as fp16 (the reference's fall-through, LF/src/utils.cpp:1303-1318)
    mil.nnopt_unregister_weight(qb)
    Wf = mil.Buffer.from_host(W)
    assert mil.pytorch_linear(queue, 1, N, K, xb, Wf, ob)
    queue.finish()
    assert np.array_equal(ob.read(np.uint16, (N,)), O.gemv_f16(x, W))
    # gate/up with mixed kinds is "not taken"
    assert mil.nnopt_register_int8_weight(qb, sb, N, K)
    assert not mil.fused_gate_up_silu_m1(queue, N, K, xb, qb, Wf, ob)
    mil.nnopt_unregister_weight(qb)


def test_batch_and_graph_replay(queue):
    # a chain of dependent projections, replayed from a graph several times with eager work between
    K0, N0, N1 = 896, 4864, 896
    x = synth_x(24, K0)
    q0, s0 = mil.quantize_int8(synth_w(25, N0, K0))
    q1, s1 = mil.quantize_int8(synth_w(26, N1, N0))
    xb, hb, yb = mil.Buffer.from_host(x), mil.Buffer(N0 * 2), mil.Buffer(N1 * 2)
    W0, S0, W1, S1 = (mil.Buffer.from_host(a) for a in (q0, s0, q1, s1))
    assert mil.nnopt_register_int8_weight(W0, S0, N0, K0)
    assert mil.nnopt_register_int8_weight(W1, S1, N1, N0)
    calls = mil.make_calls([(1, N0, K0, xb, W0, hb), (1, N1, N0, hb, W1, yb)])
    h = O.gemv_i8(x, q0, s0.view(np.uint16))
    want = O.gemv_i8(h.view(np.float16), q1, s1.view(np.uint16))
    assert mil.linear_batch(queue, calls) == 2
    queue.finish()
    assert np.array_equal(yb.read(np.uint16, (N1,)), want)
    with mil.Graph(queue) as g:
        assert mil.linear_batch(queue, calls) == 2
    for rep in range(3):
        yb.write(np.zeros(N1, np.uint16))
        hb.write(np.zeros(N0, np.uint16))
        g.launch()
        queue.finish()
        assert np.array_equal(yb.read(np.uint16, (N1,)), want), f"replay {rep}"
    for b in (W0, W1):
        mil.nnopt_unregister_weight(b)


@pytest.mark.parametrize("kind", ["i8", "q4", "f16"])
def test_batch_merges_independent_calls_bit_exact(queue, kind):
    """q/k/v-style calls (same x, different W and out) go out as one launch; the results must
    equal separate calls, and calls that depend on each other must still run in order."""
    K = 896
    Ns = [896, 128, 128, 36, 4864]                  # five calls: more than one launch can hold
    x = synth_x(40, K)
    xb = mil.Buffer.from_host(x)
    keep, calls, wants = [], [], []
    for i, N in enumerate(Ns):
        W = synth_w(41 + i, N, K)
        ob = mil.Buffer.from_host(np.zeros(N, np.uint16))
        if kind == "i8":
            q, s = mil.quantize_int8(W)
            Wb, sb = mil.Buffer.from_host(q), mil.Buffer.from_host(s)
            assert mil.nnopt_register_int8_weight(Wb, sb, N, K)
            wants.append(O.gemv_i8(x, q, s.view(np.uint16)))
        elif kind == "q4":
            p, sc = mil.quantize_q4(W)
            Wb, sb = mil.Buffer.from_host(p), mil.Buffer.from_host(sc)
            assert mil.nnopt_register_q4_weight(Wb, sb, N, K)
            wants.append(O.gemv_q4(x, p, sc.view(np.uint16)))
        else:
            Wb, sb = mil.Buffer.from_host(W), None
            wants.append(O.gemv_f16(x, W))
        keep += [Wb, sb, ob]
        calls.append((1, N, K, xb, Wb, ob))
    arr = mil.make_calls(calls)
    assert mil.linear_batch(queue, arr) == 5
    queue.finish()
    for (_, N, _, _, _, ob), want in zip(calls, wants):
        assert np.array_equal(ob.read(np.uint16, (N,)), want)
    for b in keep:
        if b is not None:
            mil.nnopt_unregister_weight(b)


def test_batch_keeps_dependent_calls_in_order(queue):
    K = 896
    x = synth_x(60, K)
    Wa, Wb_ = synth_w(61, K, K), synth_w(62, K, K)
    qa, sa = mil.quantize_int8(Wa)
    qb, sb = mil.quantize_int8(Wb_)
    xb, hb, yb = mil.Buffer.from_host(x), mil.Buffer(K * 2), mil.Buffer(K * 2)
    A, SA, B, SB = (mil.Buffer.from_host(a) for a in (qa, sa, qb, sb))
    assert mil.nnopt_register_int8_weight(A, SA, K, K) and mil.nnopt_register_int8_weight(B, SB, K, K)
    # second call reads the first call's output; third reads x again but writes where the
    # second reads (write-after-read): order must be kept
    calls = mil.make_calls([(1, K, K, xb, A, hb), (1, K, K, hb, B, yb), (1, K, K, xb, B, hb)])
    assert mil.linear_batch(queue, calls) == 3
    queue.finish()
    h = O.gemv_i8(x, qa, sa.view(np.uint16))
    assert np.array_equal(yb.read(np.uint16, (K,)), O.gemv_i8(h.view(np.float16), qb, sb.view(np.uint16)))
    assert np.array_equal(hb.read(np.uint16, (K,)), O.gemv_i8(x, qb, sb.view(np.uint16)))
    mil.nnopt_unregister_weight(A)
    mil.nnopt_unregister_weight(B)


@pytest.mark.parametrize("kind", ["i8", "q4"])
def test_lm_head_full_size(queue, kind):
    """Config 3: W[151936 x 896].  Bit-exact against the oracle on every row."""
    N, K = 151936, 896
    print(f"lm_head {kind}", flush=True)
    W, x = synth_w(27, N, K), synth_x(28, K)
    if kind == "i8":
        q, s = mil.quantize_int8(W)
        got = _run_linear(queue, 1, N, K, x, q, s, "i8")[0]
        want = O.gemv_i8(x, q, s.view(np.uint16))
    else:
        p, sc = mil.quantize_q4(W)
        got = _run_linear(queue, 1, N, K, x, p, sc, "q4")[0]
        want = O.gemv_q4(x, p, sc.view(np.uint16))
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {N} differ"
    # against the unquantised product the quantisation error stays small: cosine bar only
    ref = (W.astype(np.float32) @ x.astype(np.float32))
    g = got.view(np.float16).astype(np.float32)
    cos = float(np.dot(g, ref) / (np.linalg.norm(g) * np.linalg.norm(ref)))
    assert cos > (0.999 if kind == "i8" else 0.98)
    assert_tolerance(got.view(np.float16), want.view(np.float16))
