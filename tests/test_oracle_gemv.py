"""GEMV arithmetic of the oracle, checked against what the mathematics and the
kernel sources fix.

The reference holds no known-answer vector for any GEMV kernel, so these pins
are: unit vectors (a wrong index or a dropped K tail fails), exactly summable
integer data (a dropped term or wrong scale fails), an fp64 dot product within
the stated tolerance, and cancellation probes that expose the lane ownership
(k = 256j + 4t) and the 64-lane tree pairing (t with t+s, s = 32..1) spelled
out in QW/kernels/gemv_m1.cl:386-424, LF/kernels/gemv_m1_int8.cl:46-68 and
LF/kernels/gemv_m1_q4.cl:59-116."""
import numpy as np
import pytest

import oracle_lib as O

SHAPES = [(8, 256), (12, 576), (16, 896), (8, 1024), (4, 4864), (20, 64), (5, 36)]


def _rand(N, K, seed):
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    x = rng.standard_normal(K).astype(np.float16)
    return W, x


def _check_tol(got_u16, want64):
    got = O.f16(got_u16).astype(np.float64)
    err = np.abs(got - want64)
    assert np.all(err <= 1e-3 + 1e-3 * np.abs(want64))
    cos = np.dot(got, want64) / (np.linalg.norm(got) * np.linalg.norm(want64))
    assert cos >= 0.9999


@pytest.mark.parametrize("N,K", SHAPES)
def test_f16_vs_fp64(N, K):
    W, x = _rand(N, K, 10)
    _check_tol(O.gemv_f16(x, W), W.astype(np.float64) @ x.astype(np.float64))


@pytest.mark.parametrize("N,K", SHAPES)
def test_i8_vs_fp64(N, K):
    W, x = _rand(N, K, 11)
    q, s = O.quantize_int8(W)
    want = (q.astype(np.float64) @ x.astype(np.float64)) * O.f16(s).astype(np.float64)
    _check_tol(O.gemv_i8(x, q, s), want)


@pytest.mark.parametrize("N,K", [(8, 256), (16, 896), (8, 1024), (4, 4864), (6, 32), (6, 96)])
def test_q4_vs_fp64(N, K):
    W, x = _rand(N, K, 12)
    p, sc = O.quantize_q4(W)
    wf = np.empty((N, K), np.float32)
    O.lib.orc_dequant_q4_to_f32(p, sc, N, K, wf)
    _check_tol(O.gemv_q4(x, p, sc), wf.astype(np.float64) @ x.astype(np.float64))


@pytest.mark.parametrize("K", [576, 896, 4864])
def test_unit_vectors_return_columns(K):
    N = 8
    W, _ = _rand(N, K, 13)
    q, s = O.quantize_int8(W)
    p, sc = O.quantize_q4(W)
    wq4 = np.empty((N, K), np.float32)
    O.lib.orc_dequant_q4_to_f32(p, sc, N, K, wq4)
    for k in [0, 1, 3, 4, 255, 256, K // 2 + 1, K - 129, K - 5, K - 1]:
        x = np.zeros(K, np.float16)
        x[k] = 1.0
        assert np.array_equal(O.f16(O.gemv_f16(x, W)), W[:, k])
        want = (q[:, k].astype(np.float32) * O.f16(s).astype(np.float32)).astype(np.float16)
        assert np.array_equal(O.f16(O.gemv_i8(x, q, s)), want)
        assert np.array_equal(O.f16(O.gemv_q4(x, p, sc)), wq4[:, k].astype(np.float16))


def test_exact_integer_sums():
    # |sums| stay below 2^24, so every fp32 order gives the same value
    rng = np.random.default_rng(14)
    N, K = 16, 896
    q = rng.integers(-127, 128, (N, K)).astype(np.int8)
    x = rng.integers(-4, 5, K).astype(np.float16)
    s = (2.0 ** rng.integers(-12, -6, N)).astype(np.float16).view(np.uint16)
    want = ((q.astype(np.int64) @ x.astype(np.int64)).astype(np.float64) * O.f16(s)).astype(np.float16)
    assert np.array_equal(O.f16(O.gemv_i8(x, q, s)), want)

    p = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    sc = (2.0 ** rng.integers(-8, -3, (N, K // 32))).astype(np.float16).view(np.uint16)
    nib = np.stack([p & 15, p >> 4], -1).reshape(N, K).astype(np.int64) - 8
    wd = nib * np.repeat(O.f16(sc).astype(np.float64), 32, axis=1)
    want = (wd @ x.astype(np.float64)).astype(np.float16)
    assert np.array_equal(O.f16(O.gemv_q4(x, p, sc)), want)

    Wf = rng.integers(-64, 65, (N, K)).astype(np.float16)
    want = (Wf.astype(np.int64) @ x.astype(np.int64)).astype(np.float16)
    assert np.array_equal(O.f16(O.gemv_f16(x, Wf)), want)


def _probe_f16(K, big_at, one_at, neg_at):
    """x*w = +2^24 at big_at, +1 at one_at, -2^24 at neg_at."""
    W = np.zeros((1, K), np.float16)
    x = np.zeros(K, np.float16)
    for k, (xv, wv) in ((big_at, (4096.0, 4096.0)), (one_at, (1.0, 1.0)), (neg_at, (4096.0, -4096.0))):
        x[k], W[0, k] = xv, wv
    return float(O.f16(O.gemv_f16(x, W))[0])


def test_lane_ownership_probe_f16():
    K = 896
    # same lane, same iteration (k = 0 and 2): the 1 is absorbed by 2^24 before the
    # cancelling term, which lives in another lane, arrives -> 0
    assert _probe_f16(K, 0, 2, 8) == 0.0
    # cancelling pair inside one lane (k = 0, 1), the 1 in the next lane (k = 4) -> survives
    assert _probe_f16(K, 0, 4, 1) == 1.0
    # k and k+256 belong to the same lane (next iteration): absorbed again
    assert _probe_f16(K, 0, 256, 8) == 0.0
    # the K tail (k >= 768) is owned by lanes 0..31: k=768 is lane 0 again
    assert _probe_f16(K, 0, 768, 8) == 0.0
    assert _probe_f16(K, 768, 4, 0) == 1.0


def test_tree_pairing_probe_f16():
    K = 256                                    # one iteration, lane t <-> k = 4t
    lane = lambda t: 4 * t
    # first tree step pairs t with t+32: big in 0, -big in 32 cancel at once, 1 in lane 1 survives
    assert _probe_f16(K, lane(0), lane(1), lane(32)) == 1.0
    # 1 sits in lane 32 (joins lane 0 first and is absorbed), -big in lane 16 arrives one step later
    assert _probe_f16(K, lane(0), lane(32), lane(16)) == 0.0
    # big in 0, 1 in lane 16 (joins at s=16), -big in lane 32 (joins at s=32, before) -> survives
    assert _probe_f16(K, lane(0), lane(16), lane(32)) == 1.0
    # last step pairs lane 0 with lane 1
    # lane 2 joins lane 0 at s=2 (cancelling), lane 1 joins at s=1 -> survives
    assert _probe_f16(K, lane(0), lane(1), lane(2)) == 1.0


def test_scale_applied_after_reduction_i8():
    # int8: y = fp16(s * sum).  With s = 2^-10 and sum = 2049 the product 2.0009765625
    # rounds to 2.0; scaling each term first would give the same here, so use a sum that
    # only fits fp32 when unscaled: sum = 2^24 + 2 is exact, times 2^-24 -> fp16(1.0000001) = 1
    K = 256
    q = np.zeros((1, K), np.int8)
    x = np.zeros(K, np.float16)
    q[0, 0], x[0] = 127, 2048.0        # lane 0
    q[0, 4], x[4] = 127, 2048.0        # lane 1
    q[0, 8], x[8] = 1, 3.0             # lane 2
    s = np.array([2.0 ** -8], np.float16).view(np.uint16)
    want = np.float16(np.float32(127 * 2048 * 2 + 3) * np.float32(2.0 ** -8))
    assert O.f16(O.gemv_i8(x, q, s))[0] == want


def test_q4_block_scale_and_pixel_probe():
    K = 896
    p = np.full((1, K // 2), 0x88, np.uint8)          # every weight 0
    sc = np.zeros((1, K // 32), np.float16)
    x = np.zeros(K, np.float16)
    # element 40 lives in pixel 5 (lane 5), scale block 1; element 41 the high nibble of the same byte
    p[0, 20] = (8 + 3) | ((8 - 5) << 4)
    sc[0, 1] = 0.5
    sc[0, 0] = 64.0                                   # a wrong block index would show
    sc[0, 2] = 64.0
    x[40], x[41] = 2.0, 1.0
    got = O.f16(O.gemv_q4(x, p, sc.view(np.uint16)))[0]
    assert got == np.float16((2 * 3 + 1 * -5) * 0.5)
    # tail pixel: element 895 is the high nibble of byte 447, pixel 111 = iteration 1, lane 47, block 27
    p[0, 447] = 0x08 | ((8 + 7) << 4)
    sc[0, 27] = 0.25
    x[:] = 0
    x[895] = 4.0
    got = O.f16(O.gemv_q4(x, p, sc.view(np.uint16)))[0]
    assert got == np.float16(7 * 4 * 0.25)


def test_q4_inner_sum_is_per_pixel_then_scaled():
    # d = sum over the 8 elements of a pixel in fp32, then acc = fma(d, scale, acc).
    # Within one pixel: +2^24 (7*... not reachable with |w|<=8), so use x = 2^15 * 2^... :
    # x = 32768 (fp16), w = -8 (nibble 0) -> -2^18 ; build 2^24 from 64 such terms is not
    # possible in one pixel, so probe with the scale instead: d = 1 + (-1) exactly 0 inside
    # a pixel regardless of scale, while a neighbouring pixel contributes 3*s.
    K = 64
    p = np.full((1, K // 2), 0x88, np.uint8)
    sc = np.array([[0.1, 0.3]], np.float16)
    x = np.zeros(K, np.float16)
    p[0, 0] = (8 + 1) | ((8 - 1) << 4)      # elements 0,1 = +1,-1 (pixel 0)
    x[0] = x[1] = 1000.0
    p[0, 4] = (8 + 3) | (8 << 4)            # element 8 = +3 (pixel 1)
    x[8] = 1.0
    got = O.f16(O.gemv_q4(x, p, sc.view(np.uint16)))[0]
    assert got == np.float16(np.float32(3.0) * np.float16(0.1).astype(np.float32))


def test_fused_epilogues():
    rng = np.random.default_rng(15)
    N, K = 24, 576
    W, x = _rand(N, K, 16)
    Wu, _ = _rand(N, K, 17)
    q, s = O.quantize_int8(W)
    qu, su = O.quantize_int8(Wu)
    res0 = rng.standard_normal(N).astype(np.float16)
    xs = O.u16(x)

    y32 = np.empty(N, np.float32)
    O.lib.orc_gemv_i8_f32(xs, q, s, y32, N, K)
    res = O.u16(res0).copy()
    O.lib.orc_gemv_i8_add(xs, q, s, res, N, K)
    want = (y32.astype(np.float64) + res0.astype(np.float64))
    assert np.all(np.abs(O.f16(res).astype(np.float64) - want) <= np.abs(want) * 2**-10 + 1e-7)

    res = O.u16(res0).copy()
    O.lib.orc_gemv_f16_add(xs, O.u16(W), res, N, K)
    want = W.astype(np.float64) @ x.astype(np.float64) + res0.astype(np.float64)
    assert np.all(np.abs(O.f16(res).astype(np.float64) - want) <= np.abs(want) * 2**-10 + 1e-5)

    out = np.empty(N, np.uint16)
    O.lib.orc_gate_up_silu_i8(xs, q, qu, s, su, out, N, K)
    g = (q.astype(np.float64) @ x.astype(np.float64)) * O.f16(s)
    u = (qu.astype(np.float64) @ x.astype(np.float64)) * O.f16(su)
    want = g / (1 + np.exp(-g)) * u
    assert np.all(np.abs(O.f16(out).astype(np.float64) - want) <= np.abs(want) * 2**-9 + 1e-5)

    O.lib.orc_gate_up_silu_f16(xs, O.u16(W), O.u16(Wu), out, N, K)
    g = W.astype(np.float64) @ x.astype(np.float64)
    u = Wu.astype(np.float64) @ x.astype(np.float64)
    want = g / (1 + np.exp(-g)) * u
    assert np.all(np.abs(O.f16(out).astype(np.float64) - want) <= np.abs(want) * 2**-9 + 1e-5)


def test_silu_gate_epilogue_closed_form():
    """gate = fp16(silu(gate) * (W x)) against float64, for the three weight kinds; and the special
    cases that pin the operand roles: gate = 0 gives 0 whatever W x is, a large gate passes W x
    times gate through (sigmoid -> 1), W x = 0 gives 0."""
    rng = np.random.default_rng(25)
    N, K = 24, 1024
    W, x = _rand(N, K, 26)
    q, s = O.quantize_int8(W)
    p, sc = O.quantize_q4(W)
    gate0 = (rng.standard_normal(N) * 2).astype(np.float16)
    xs = O.u16(x)
    sig = lambda g: g / (1 + np.exp(-g))
    x64, g64 = x.astype(np.float64), gate0.astype(np.float64)

    gate = O.u16(gate0).copy()
    O.lib.orc_gemv_f16_silu_gate(xs, O.u16(W), gate, N, K)
    want = sig(g64) * (W.astype(np.float64) @ x64)
    assert np.all(np.abs(O.f16(gate).astype(np.float64) - want) <= np.abs(want) * 2**-9 + 1e-5)

    gate = O.u16(gate0).copy()
    O.lib.orc_gemv_i8_silu_gate(xs, q, s, gate, N, K)
    want = sig(g64) * ((q.astype(np.float64) @ x64) * O.f16(s))
    assert np.all(np.abs(O.f16(gate).astype(np.float64) - want) <= np.abs(want) * 2**-9 + 1e-5)

    gate = O.u16(gate0).copy()
    O.lib.orc_gemv_q4_silu_gate(xs, p, np.ascontiguousarray(sc), gate, N, K)
    wq4 = np.empty((N, K), np.float32)
    O.lib.orc_dequant_q4_to_f32(p, np.ascontiguousarray(sc), N, K, wq4)
    want = sig(g64) * (wq4.astype(np.float64) @ x64)
    assert np.all(np.abs(O.f16(gate).astype(np.float64) - want) <= np.abs(want) * 2**-9 + 1e-5)

    zero = np.zeros(N, np.uint16)
    O.lib.orc_gemv_f16_silu_gate(xs, O.u16(W), zero, N, K)
    assert not (zero & 0x7FFF).any()                            # silu(0) = 0 (of either sign)
    big = O.u16(np.full(N, 30.0, np.float16)).copy()
    O.lib.orc_gemv_f16_silu_gate(xs, O.u16(W), big, N, K)       # sigmoid(30) rounds to 1 in fp32
    y = np.empty(N, np.float64)
    want = (30.0 * (W.astype(np.float64) @ x64))
    assert np.all(np.abs(O.f16(big).astype(np.float64) - want) <= np.abs(want) * 2**-10 + 1e-6)
    gate = O.u16(gate0).copy()
    O.lib.orc_gemv_f16_silu_gate(O.u16(np.zeros(K, np.float16)), O.u16(W), gate, N, K)
    assert not (gate & 0x7FFF).any()                            # W x = 0


def test_gemm_rows_are_gemvs():
    M, N, K = 5, 12, 896
    rng = np.random.default_rng(18)
    W, _ = _rand(N, K, 19)
    X = rng.standard_normal((M, K)).astype(np.float16)
    q, s = O.quantize_int8(W)
    p, sc = O.quantize_q4(W)
    out = O.gemm_i8(X, q, s)
    for m in range(M):
        assert np.array_equal(out[m], O.gemv_i8(X[m], q, s))
    out = O.gemm_q4(X, p, sc)
    assert np.array_equal(out[3], O.gemv_q4(X[3], p, sc))
    out = O.gemm_f16(X, W)
    assert np.array_equal(out[4], O.gemv_f16(X[4], W))


def test_threads_do_not_change_bits():
    W, x = _rand(64, 896, 20)
    q, s = O.quantize_int8(W)
    assert np.array_equal(O.gemv_i8(x, q, s, threads=1), O.gemv_i8(x, q, s, threads=O.THREADS))


@pytest.mark.parametrize("N,K", [(24, 1024), (16, 896), (5, 4864), (7, 96)])
def test_q4_residual_add_epilogue(N, K):
    """orc_gemv_q4_add: the reference has an int8 residual kernel only (SM/kernels/block_fused_int8.cl:105-174),
    so the mathematics pins the Q4 form: res + dequant(W) x in float64 within one fp16 step (a subtracted or
    dropped residual, a residual added after the rounding of the product, a wrong row's residual all fail:
    the residuals are large against the products and differ per row), a zero residual gives orc_gemv_q4's
    bits (x + 0 is x in fp32), and a residual that swamps the product comes back unchanged."""
    rng = np.random.default_rng(31 + K)
    W, x = _rand(N, K, 32 + N)
    p, sc = O.quantize_q4(W)
    sc = np.ascontiguousarray(sc)
    xs = O.u16(x)
    wf = np.empty((N, K), np.float32)
    O.lib.orc_dequant_q4_to_f32(p, sc, N, K, wf)
    prod = wf.astype(np.float64) @ x.astype(np.float64)

    res0 = (rng.standard_normal(N) * 3 + np.arange(N)).astype(np.float16)
    res = O.u16(res0).copy()
    O.lib.orc_gemv_q4_add(xs, p, sc, res, N, K)
    want = prod + res0.astype(np.float64)
    got = O.f16(res).astype(np.float64)
    # one fp16 step at the result's size (2^-10 relative), plus the fp32 accumulation error of the sum
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0**-10 + 1e-5)
    # the tolerance separates it from the two-rounding form only on average, so also: most outputs are
    # the correctly rounded fp16 of the fp64 value
    exact = want.astype(np.float16).astype(np.float64)
    assert np.mean(got == exact) >= 0.9

    zero = np.zeros(N, np.uint16)
    O.lib.orc_gemv_q4_add(xs, p, sc, zero, N, K)
    assert np.array_equal(zero, O.gemv_q4(x, p, sc))

    big = O.u16(np.full(N, 60000.0, np.float16)).copy()
    O.lib.orc_gemv_q4_add(xs, p, sc, big, N, K)
    assert np.all(np.abs(O.f16(big).astype(np.float64) - (60000.0 + prod)) <= 32.0)   # one fp16 step at 6e4
    assert np.all(np.isfinite(O.f16(big)))
