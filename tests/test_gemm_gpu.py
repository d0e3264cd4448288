"""GPU parity of the prefill GEMM (M > 1 on the matrix cores), through the C ABI.

Reference semantics: row i of out is the GEMV of row i of x (the reference's quantised
prefill is a loop of M = 1 calls, LF/src/model.cpp:243-250).  The MFMA kernel sums in a
different fp32 order than the GEMV kernels, so the bar here is the stated tolerance
(max-abs/rel 1e-3, cosine >= 0.9999), tightened to "at most 1 fp16 ulp apart"; the batched
GEMV mode of the same entry point stays bit-exact."""
import numpy as np
import pytest

import oracle_lib as O
from helpers import assert_tolerance, mil, synth_w, synth_x

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def queue():
    assert mil.lib().mi_init(0) == 1, "no gfx950 device"
    q = mil.Queue()
    yield q
    q.finish()


def _ulp_apart(a_u16, b_u16):
    """|a - b| in units of the fp16 spacing at max(|b|, 1e-3 max|b|): outputs that cancel to
    almost zero carry the absolute fp32 rounding error of sums of much larger terms, so their
    own (tiny) fp16 spacing is not the yardstick."""
    a = a_u16.view(np.float16).astype(np.float64)
    b = b_u16.view(np.float16).astype(np.float64)
    mag = np.maximum(np.abs(b), 1e-3 * np.abs(b).max())
    step = np.spacing(mag.astype(np.float16)).astype(np.float64)
    return np.abs(a - b) / step


def _gemm(queue, M, N, K, X, W_host, scale_host, kind, tile=0, plan=None):
    """tile is the mi_set_gemm_mode value: 0 = the library's own choice, 1 = rows of GEMV,
    2 = the 64 x 64 MFMA kernel, 3 = the wide kernel with its own choice of rows of x per
    block, 30 = the kernel with 256 x 256 blocks (int8), 4 = Q4 weights rounded to fp16 once, 5 = the streaming kernel for up to 64 rows of x,
    11..15 = the wide kernel with 32, 64, .. 160 rows of x per block.  plan: a list that receives (kernel, rows of x per block, slices of K) of the call."""
    xb, wb = mil.Buffer.from_host(X), mil.Buffer.from_host(W_host)
    sb = mil.Buffer.from_host(scale_host) if scale_host is not None else None
    if kind == "i8":
        assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    elif kind == "q4":
        assert mil.nnopt_register_q4_weight(wb, sb, N, K)
    pad = 128
    guard = np.full(M * N + 2 * pad, 0x7BCD, np.uint16)
    ob = mil.Buffer.from_host(guard)
    mil.lib().mi_set_gemm_mode(tile)
    try:
        if plan is not None:
            plan.append(mil.linear_plan(queue, M, N, K, xb, wb))
        assert mil.pytorch_linear(queue, M, N, K, xb, wb, ob.ptr + 2 * pad)
        queue.finish()
    finally:
        mil.lib().mi_set_gemm_mode(0)
    full = ob.read(np.uint16, guard.shape)
    assert np.all(full[:pad] == 0x7BCD) and np.all(full[-pad:] == 0x7BCD), "wrote outside out[M,N]"
    mil.nnopt_unregister_weight(wb)
    return full[pad:-pad].reshape(M, N)


@pytest.mark.parametrize("tile", [0, 2, 3, 11, 12, 13, 14, 15, 30])
@pytest.mark.parametrize("M", [16, 64, 100, 512])
@pytest.mark.parametrize("N,K", [(4864, 896), (896, 4864), (200, 128), (130, 576), (131, 64)])
def test_int8_gemm_matches_rows_of_gemv(queue, M, N, K, tile):
    print(f"int8 gemm M={M} N={N} K={K} tile mode {tile}", flush=True)
    W, X = synth_w(700 + N, N, K), synth_x(800 + M, M, K)
    q, s = mil.quantize_int8(W)
    got = _gemm(queue, M, N, K, X, q, s, "i8", tile)
    want = O.gemm_i8(X, q, s.view(np.uint16))
    assert_tolerance(got.view(np.float16), want.view(np.float16))
    d = _ulp_apart(got, want)
    assert d.max() <= 1, f"max {d.max()} fp16 steps apart"
    assert np.mean(got == want) > 0.99


@pytest.mark.parametrize("tile", [0, 2, 3, 11, 12, 13, 14, 15])
@pytest.mark.parametrize("M,N,K", [(64, 4864, 896), (256, 896, 4864), (33, 200, 128), (130, 131, 64), (16, 1536, 576),
                                   (2048, 4864, 128)])
def test_fp16_gemm_matches_rows_of_gemv(queue, M, N, K, tile):
    print(f"fp16 gemm M={M} N={N} K={K} tile mode {tile}", flush=True)
    W, X = synth_w(900 + N, N, K), synth_x(901 + M, M, K)
    got = _gemm(queue, M, N, K, X, W, None, "f16", tile)
    want = O.gemm_f16(X, W)
    assert_tolerance(got.view(np.float16), want.view(np.float16))
    assert _ulp_apart(got, want).max() <= 1


@pytest.mark.parametrize("tile", [2, 3, 11, 12, 13, 14, 15])
def test_fp16_gemm_exact_and_repeatable_on_integer_data(queue, tile):
    """Small integers in both operands: every sum is exact, so the result is that of integer
    arithmetic whatever the order; and 10 launches of the same call give the same bits."""
    rng = np.random.default_rng(7)
    M, N, K = 100, 520, 1024
    W = rng.integers(-8, 9, (N, K)).astype(np.float16)
    X = rng.integers(-3, 4, (M, K)).astype(np.float16)
    want = (X.astype(np.int64) @ W.astype(np.int64).T).astype(np.float16)
    for _ in range(10):
        got = _gemm(queue, M, N, K, X, W, None, "f16", tile)
        assert np.array_equal(got.view(np.float16), want)


@pytest.mark.parametrize("tile", [2, 3, 11, 13, 15, 30])
def test_gemm_exact_on_integer_data(queue, tile):
    # small integers: every partial sum is exact in fp32, so any summation order gives the same bits
    rng = np.random.default_rng(3)
    M, N, K = 96, 192, 256
    q = rng.integers(-127, 128, (N, K)).astype(np.int8)
    X = rng.integers(-3, 4, (M, K)).astype(np.float16)
    s = (2.0 ** rng.integers(-10, -6, N)).astype(np.float16)
    got = _gemm(queue, M, N, K, X, q, s, "i8", tile)
    want = ((X.astype(np.int64) @ q.astype(np.int64).T).astype(np.float64) * s.astype(np.float64)).astype(np.float16)
    assert np.array_equal(got.view(np.float16), want)
    assert np.array_equal(got, O.gemm_i8(X, q, s.view(np.uint16)))


@pytest.mark.parametrize("tile", [2, 3, 12, 14, 15, 30])
def test_gemm_unit_rows_pick_weight_columns(queue, tile):
    # x rows are unit vectors: out[i, :] must be the dequantised column k_i of W (index check)
    M, N, K = 64, 320, 896
    W = synth_w(910, N, K)
    q, s = mil.quantize_int8(W)
    ks = (np.arange(M) * 37 + 5) % K
    X = np.zeros((M, K), np.float16)
    X[np.arange(M), ks] = 1.0
    got = _gemm(queue, M, N, K, X, q, s, "i8", tile).view(np.float16)
    want = (q[:, ks].T.astype(np.float32) * s.astype(np.float32)[None, :]).astype(np.float16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("tile", [2, 11, 12, 13, 14, 15, 30])
def test_gemm_repeats_identically(queue, tile):
    """The same launch 25 times: every result identical to the first and within tolerance of the
    oracle (a race between the LDS fills, the fragment reads and the barriers would show here)."""
    M, N, K = 100, 1000, 1024
    print(f"repeat tile mode {tile}", flush=True)
    W, X = synth_w(940, N, K), synth_x(941, M, K)
    q, s = mil.quantize_int8(W)
    want = O.gemm_i8(X, q, s.view(np.uint16))
    xb, wb, sb = mil.Buffer.from_host(X), mil.Buffer.from_host(q), mil.Buffer.from_host(s)
    assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    outs = [mil.Buffer(M * N * 2) for _ in range(25)]
    mil.lib().mi_set_gemm_mode(tile)
    try:
        for ob in outs:
            assert mil.pytorch_linear(queue, M, N, K, xb, wb, ob)
        queue.finish()
    finally:
        mil.lib().mi_set_gemm_mode(0)
    first = outs[0].read(np.uint16, (M, N))
    assert_tolerance(first.view(np.float16), want.view(np.float16))
    for i, ob in enumerate(outs[1:]):
        assert np.array_equal(ob.read(np.uint16, (M, N)), first), f"launch {i + 1} differs from launch 0"
    mil.nnopt_unregister_weight(wb)


def test_the_256_row_blocks_give_the_wide_kernels_bits_and_are_the_choice_for_large_contractions(queue):
    """The kernel with 256 x 256 blocks (128 x 128 per wavefront) feeds every output element the same K-stages
    in the same order as the wide kernel, so the two agree bit for bit: ragged shapes with partial blocks in
    both directions (mode 30 against mode 15, guard words intact), then a contraction large enough for the
    library to take the kernel by itself (8192 x 8192 x 2048: 1024 blocks, four rounds), whose plan is checked
    and whose output is compared with the wide kernel's through a row sample and a checksum of every row."""
    for (M, N, K) in ((700, 1300, 2112), (257, 255, 64), (1024, 1024, 2048), (3, 600, 128)):
        print(f"256-row blocks M={M} N={N} K={K}", flush=True)
        W, X = synth_w(960 + M, N, K), synth_x(961 + M, M, K)
        q, s = mil.quantize_int8(W)
        plan = []
        got = _gemm(queue, M, N, K, X, q, s, "i8", 30, plan=plan)
        assert plan[0][0] == 5 and plan[0][1] == 256, plan
        assert np.array_equal(got, _gemm(queue, M, N, K, X, q, s, "i8", 15))
    M, N, K = 8192, 8192, 2048
    print(f"256-row blocks M={M} N={N} K={K}, the library's own choice", flush=True)
    W, X = synth_w(970, N, K), synth_x(971, M, K)
    q, s = mil.quantize_int8(W)
    xb, wb, sb = mil.Buffer.from_host(X), mil.Buffer.from_host(q), mil.Buffer.from_host(s)
    assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    outs = []
    try:
        assert mil.linear_plan(queue, M, N, K, xb, wb)[0] == 5
        for mode in (0, 15):
            ob = mil.Buffer(M * N * 2)
            mil.lib().mi_set_gemm_mode(mode)
            assert mil.pytorch_linear(queue, M, N, K, xb, wb, ob)
            queue.finish()
            outs.append(ob.read(np.uint16, (M, N)))
    finally:
        mil.lib().mi_set_gemm_mode(0)
        mil.nnopt_unregister_weight(wb)
    assert np.array_equal(outs[0], outs[1])
    rows = [0, 255, 256, 4097, 8191]                     # and against the oracle, on a few rows
    want = O.gemm_i8(X[rows], q, s.view(np.uint16))
    assert _ulp_apart(outs[0][rows], want).max() <= 1


# ---- up to 64 rows of x: the kernel that streams W once (mode 5; mode 0 picks it by itself) ----

@pytest.mark.parametrize("kind", ["i8", "f16", "q4"])
@pytest.mark.parametrize("M", [2, 7, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(4864, 896), (896, 4864), (130, 576), (131, 64), (16, 64), (1000, 1024), (20000, 128),
                                 (520, 192), (1024, 4608)])
def test_streaming_gemm_few_rows(queue, kind, M, N, K):
    """(Q4: an iteration is 128 values of K; at K = 64, 192, 576 half of the lanes sit the last one out.)"""
    print(f"{kind} streaming gemm M={M} N={N} K={K}", flush=True)
    W, X = synth_w(1700 + N, N, K), synth_x(1800 + M, M, K)
    plan = []
    if kind == "i8":
        q, s = mil.quantize_int8(W)
        got = _gemm(queue, M, N, K, X, q, s, "i8", 5, plan)
        want = O.gemm_i8(X, q, s.view(np.uint16))
    elif kind == "q4":
        p, s = mil.quantize_q4(W)
        got = _gemm(queue, M, N, K, X, p, s, "q4", 5, plan)
        want = O.gemm_q4(X, p, s.view(np.uint16))
        wt = _q4_values(p).astype(np.float64) * np.repeat(s.astype(np.float64), 32, axis=1)
        exact = (X.astype(np.float64) @ wt.T).astype(np.float16)
        assert _ulp_apart(got, exact.view(np.uint16)).max() <= 1      # the weights entered exactly: one rounding from the true sum
    else:
        got = _gemm(queue, M, N, K, X, W, None, "f16", 5, plan)
        want = O.gemm_f16(X, W)
    kernel, rows, slices = plan[0]
    assert kernel == 4 and rows == 16 * ((M + 15) // 16) and slices in (1, 2, 4, 8, 16, 32)
    assert_tolerance(got.view(np.float16), want.view(np.float16))
    assert _ulp_apart(got, want).max() <= 1
    assert np.mean(got == want) > 0.99


def _streaming_q4(queue, M, N, K, X, p, s, kind):
    """Q4 through the streaming kernel: two exact terms (mode 5), or each weight rounded to fp16 once
    (mode 4, at a shape where mode 4 takes the streaming kernel by itself)."""
    if kind == "q4":
        return _gemm(queue, M, N, K, X, p, s, "q4", 5)
    plan = []
    got = _gemm(queue, M, N, K, X, p, s, "q4", 4, plan)
    assert plan[0][0] == 4, plan
    return got


def test_streaming_gemm_is_the_choice_for_a_few_rows_and_refuses_more_than_64(queue):
    N, K = 1024, 512
    W = synth_w(1900, N, K)
    q, s = mil.quantize_int8(W)
    for M, kernel in ((16, 4), (32, 4), (48, 4), (49, None), (64, None), (65, None)):
        plan = []
        _gemm(queue, M, N, K, synth_x(1901, M, K), q, s, "i8", 0, plan)
        assert (plan[0][0] == 4) == (kernel == 4), plan
    xb, wb, sb = mil.Buffer.from_host(synth_x(1902, 65, K)), mil.Buffer.from_host(q), mil.Buffer.from_host(s)
    ob = mil.Buffer(65 * N * 2)
    assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    mil.lib().mi_set_gemm_mode(5)
    try:
        assert not mil.pytorch_linear(queue, 65, N, K, xb, wb, ob)      # mode 5 has no kernel for 65 rows
    finally:
        mil.lib().mi_set_gemm_mode(0)
        mil.nnopt_unregister_weight(wb)


def test_streaming_gemm_is_not_the_choice_for_many_megabytes_of_weights(queue):
    """A long launch belongs to the wide kernel, which streams faster: an lm_head of 49 152 x 576 (28 MB
    of int8) at 16 rows of x takes the wide kernel, 14 592 x 896 (13 MB) still streams.  Plans only."""
    for (N, K, kernel) in ((49152, 576, 1), (14592, 896, 4)):
        wb, sb = mil.Buffer(N * K), mil.Buffer(N * 2)
        xb = mil.Buffer(16 * K * 2)
        assert mil.nnopt_register_int8_weight(wb, sb, N, K)
        try:
            plan = mil.linear_plan(queue, 16, N, K, xb, wb)
            assert plan[0] == kernel, (N, K, plan)
            if kernel == 1:
                assert plan[1] == 32, plan                  # no tile taller than the 16 rows of x need
        finally:
            mil.nnopt_unregister_weight(wb)


def test_plans_of_the_configured_prefill_shapes(queue):
    """Which kernel the library's own choice is at the benchmark's int8 shapes (plans only): the wide
    kernel in 64-row tiles at 512 x 4864 x 896, in 160-row tiles at 2048, in slices of K at N = 896, the
    streaming kernel at 16 rows, rows of GEMV for two rows of an MLP projection."""
    expect = {(512, 4864, 896): (1, 64, 1), (2048, 4864, 896): (1, 160, 1), (2048, 896, 4864): (1, 64, 2),
              (16, 4864, 896): (4, 16, 4), (2, 4864, 896): (0, 0, 1)}
    for (N, K) in ((4864, 896), (896, 4864)):
        wb, sb = mil.Buffer(N * K), mil.Buffer(N * 2)
        xb = mil.Buffer(2048 * K * 2)
        assert mil.nnopt_register_int8_weight(wb, sb, N, K)
        try:
            for (M, n, k), plan in expect.items():
                if (n, k) == (N, K):
                    assert mil.linear_plan(queue, M, N, K, xb, wb) == plan, (M, N, K, mil.linear_plan(queue, M, N, K, xb, wb))
        finally:
            mil.nnopt_unregister_weight(wb)


@pytest.mark.parametrize("kind", ["i8", "f16", "q4", "q4_single_rounding"])
def test_streaming_gemm_exact_on_integer_data_and_indices(queue, kind):
    """Small integers: every sum is exact whatever the order, so the result is integer arithmetic's
    (a wrong pairing of the two operands' K positions or of rows and columns cannot hide in a
    tolerance); then unit rows of x, which must pick dequantised columns of W."""
    rng = np.random.default_rng(11)
    for (M, N, K) in ((32, 528, 1024), (23, 131, 4864), (16, 4864, 896)):
        X = rng.integers(-3, 4, (M, K)).astype(np.float16)
        if kind == "i8":
            q = rng.integers(-127, 128, (N, K)).astype(np.int8)
            s = (2.0 ** rng.integers(-10, -6, N)).astype(np.float16)
            got = _gemm(queue, M, N, K, X, q, s, "i8", 5)
            want = ((X.astype(np.int64) @ q.astype(np.int64).T).astype(np.float64) * s.astype(np.float64)).astype(np.float16)
        elif kind.startswith("q4"):
            # power-of-two block scales: q * scale is an fp16 number, every product and sum exact in either mode
            p = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
            s = (2.0 ** rng.integers(-6, -2, (N, K // 32))).astype(np.float16)
            got = _streaming_q4(queue, M, N, K, X, p, s, kind)
            wt = _q4_values(p).astype(np.float64) * np.repeat(s.astype(np.float64), 32, axis=1)
            want = (X.astype(np.float64) @ wt.T).astype(np.float16)
        else:
            W = rng.integers(-8, 9, (N, K)).astype(np.float16)
            got = _gemm(queue, M, N, K, X, W, None, "f16", 5)
            want = (X.astype(np.int64) @ W.astype(np.int64).T).astype(np.float16)
        assert np.array_equal(got.view(np.float16), want), (M, N, K)
    M, N, K = 48, 320, 896
    W = synth_w(1910, N, K)
    ks = (np.arange(M) * 37 + 5) % K
    X = np.zeros((M, K), np.float16)
    X[np.arange(M), ks] = 1.0
    if kind == "i8":
        q, s = mil.quantize_int8(W)
        got = _gemm(queue, M, N, K, X, q, s, "i8", 5).view(np.float16)
        want = (q[:, ks].T.astype(np.float32) * s.astype(np.float32)[None, :]).astype(np.float16)
    elif kind.startswith("q4"):
        p, s = mil.quantize_q4(W)
        got = _streaming_q4(queue, M, N, K, X, p, s, kind).view(np.float16)
        # q * scale of column k, rounded to fp16 once (exact in two terms, the nearest fp16 in one: the same number)
        want = (_q4_values(p)[:, ks].T.astype(np.float32) * s.astype(np.float32)[:, ks // 32].T).astype(np.float16)
    else:
        got = _gemm(queue, M, N, K, X, W, None, "f16", 5).view(np.float16)
        want = W[:, ks].T
    assert np.array_equal(got, want)


def test_streaming_gemm_repeats_identically(queue):
    """25 launches of a shape whose K is shared by four blocks of eight wavefronts per strip: identical
    results (a block's slices meet in LDS and are added in slice order, not in order of arrival; the
    blocks' sums are added in index order by a second launch)."""
    M, N, K = 48, 896, 4864
    W, X = synth_w(1940, N, K), synth_x(1941, M, K)
    q, s = mil.quantize_int8(W)
    xb, wb, sb = mil.Buffer.from_host(X), mil.Buffer.from_host(q), mil.Buffer.from_host(s)
    assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    outs = [mil.Buffer(M * N * 2) for _ in range(25)]
    mil.lib().mi_set_gemm_mode(5)
    try:
        assert mil.linear_plan(queue, M, N, K, xb, wb) == (4, 48, 32)
        for ob in outs:
            assert mil.pytorch_linear(queue, M, N, K, xb, wb, ob)
        queue.finish()
    finally:
        mil.lib().mi_set_gemm_mode(0)
    first = outs[0].read(np.uint16, (M, N))
    assert_tolerance(first.view(np.float16), O.gemm_i8(X, q, s.view(np.uint16)).view(np.float16))
    for i, ob in enumerate(outs[1:]):
        assert np.array_equal(ob.read(np.uint16, (M, N)), first), f"launch {i + 1} differs from launch 0"
    mil.nnopt_unregister_weight(wb)


def _q4_values(p):
    """[N, K/2] packed bytes -> [N, K] integers in -8..7 (low nibble first)."""
    v = np.empty((p.shape[0], p.shape[1] * 2), np.int32)
    v[:, 0::2] = p & 15
    v[:, 1::2] = p >> 4
    return v - 8


@pytest.mark.parametrize("tile", [0, 3, 11, 12, 13, 14, 15])
@pytest.mark.parametrize("M", [16, 64, 100, 512])
@pytest.mark.parametrize("N,K", [(4864, 896), (896, 4864), (200, 128), (130, 576), (131, 64)])
def test_q4_gemm_matches_rows_of_gemv(queue, M, N, K, tile):
    """Q4 weights on the matrix cores.  A weight q * s (4 and 11 significant bits) is not an fp16
    number in general, so the kernel feeds it as two: q * hi + q * lo with s = hi + lo, hi the 7
    leading bits of s; both products are exact in fp16 and meet in the fp32 accumulator.  The bar
    is then the same as for int8: at most one fp16 step from the rows of GEMV."""
    print(f"q4 gemm M={M} N={N} K={K} tile mode {tile}", flush=True)
    W, X = synth_w(1700 + N, N, K), synth_x(1800 + M, M, K)
    p, s = mil.quantize_q4(W)
    got = _gemm(queue, M, N, K, X, p, s, "q4", tile)
    want = O.gemm_q4(X, p, s.view(np.uint16))
    assert_tolerance(got.view(np.float16), want.view(np.float16))
    d = _ulp_apart(got, want)
    assert d.max() <= 1, f"max {d.max()} fp16 steps apart"
    assert np.mean(got == want) > 0.99
    # and from the exact value of the sum, rounded once
    wt = _q4_values(p).astype(np.float64) * np.repeat(s.astype(np.float64), 32, axis=1)
    exact = X.astype(np.float64) @ wt.T
    assert _ulp_apart(got, exact.astype(np.float16).view(np.uint16)).max() <= 1


@pytest.mark.parametrize("M", [16, 100, 512])
@pytest.mark.parametrize("N,K", [(4864, 896), (896, 4864), (130, 576)])
def test_q4_gemm_single_rounding_mode_within_its_bound(queue, M, N, K):
    """Mode 4: a weight enters as the one fp16 number nearest to q * scale.  Checked against the
    a-priori bound of that rounding on top of one fp16 step, 2^-12 sum |w x|, and to one fp16
    step against the exact sum over the rounded weights."""
    W, X = synth_w(1700 + N, N, K), synth_x(1800 + M, M, K)
    p, s = mil.quantize_q4(W)
    got = _gemm(queue, M, N, K, X, p, s, "q4", 4)
    want = O.gemm_q4(X, p, s.view(np.uint16))
    wf = (_q4_values(p).astype(np.float32) * np.repeat(s.astype(np.float32), 32, axis=1)).astype(np.float16)
    g, w = got.view(np.float16).astype(np.float64), want.view(np.float16).astype(np.float64)
    bound = (2.0 ** -12 + 2.0 ** -20) * (np.abs(X).astype(np.float64) @ np.abs(wf).astype(np.float64).T) \
        + np.spacing(np.abs(want.view(np.float16))).astype(np.float64)
    assert np.all(np.abs(g - w) <= bound), f"worst excess {(np.abs(g - w) - bound).max()}"
    cos = np.dot(g.ravel(), w.ravel()) / (np.linalg.norm(g) * np.linalg.norm(w))
    assert cos >= 0.9999
    exact = X.astype(np.float64) @ wf.astype(np.float64).T
    assert _ulp_apart(got, exact.astype(np.float16).view(np.uint16)).max() <= 1


def test_q4_gemm_tiny_scales_keep_fp16_subnormals(queue):
    """Weights near 1e-4: the block scales and most products q * scale are fp16 subnormals.
    They must enter the sums at full value (nothing flushed to zero on the way to the matrix cores)."""
    M, N, K = 64, 512, 896
    W = (synth_w(1960, N, K).astype(np.float32) * np.float32(0.004)).astype(np.float16)
    X = (synth_x(1961, M, K).astype(np.float32) * np.float32(30.0)).astype(np.float16)
    p, s = mil.quantize_q4(W)
    assert np.mean(s.astype(np.float32) < 6.1e-5) > 0.9, "scales meant to be subnormal"
    got = _gemm(queue, M, N, K, X, p, s, "q4")
    want = O.gemm_q4(X, p, s.view(np.uint16))
    assert np.abs(want.view(np.float16).astype(np.float32)).mean() > 0.01
    assert _ulp_apart(got, want).max() <= 1


@pytest.mark.parametrize("kind", ["i8", "q4", "f16"])
@pytest.mark.parametrize("tile", [0, 2, 3])
@pytest.mark.parametrize("M", [2, 5, 15])
@pytest.mark.parametrize("N,K", [(4864, 896), (896, 4864), (130, 576)])
def test_batches_below_16_rows(queue, kind, tile, M, N, K):
    """2 <= M < 16: mode 0 picks the GEMM or M rows of GEMV by estimated time; either way, and
    with the GEMM kernels forced, the result is within one fp16 step of the rows of GEMV."""
    if kind == "q4" and tile == 2:
        pytest.skip("the 64 x 64 tiles do not take Q4 weights")
    W, X = synth_w(2700 + N, N, K), synth_x(2800 + M, M, K)
    if kind == "i8":
        q, s = mil.quantize_int8(W)
        got, want = _gemm(queue, M, N, K, X, q, s, "i8", tile), O.gemm_i8(X, q, s.view(np.uint16))
    elif kind == "q4":
        p, s = mil.quantize_q4(W)
        got, want = _gemm(queue, M, N, K, X, p, s, "q4", tile), O.gemm_q4(X, p, s.view(np.uint16))
    else:
        got, want = _gemm(queue, M, N, K, X, W, None, "f16", tile), O.gemm_f16(X, W)
    assert_tolerance(got.view(np.float16), want.view(np.float16))
    # (rows of GEMV with Q4 weights may come from the throughput kernel of the default GEMV mode,
    # whose bar is the stated tolerance)
    if not (kind == "q4" and tile == 0):
        assert _ulp_apart(got, want).max() <= 1


@pytest.mark.parametrize("tile", [3, 4, 11, 13, 15])
def test_q4_gemm_exact_on_integer_data(queue, tile):
    # power-of-two scales and small integer x: every product and partial sum is exact
    rng = np.random.default_rng(5)
    M, N, K = 96, 192, 256
    p = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    s = (2.0 ** rng.integers(-10, -6, (N, K // 32))).astype(np.float16)
    X = rng.integers(-3, 4, (M, K)).astype(np.float16)
    got = _gemm(queue, M, N, K, X, p, s, "q4", tile)
    wf = _q4_values(p).astype(np.float64) * np.repeat(s.astype(np.float64), 32, axis=1)
    want = (X.astype(np.float64) @ wf.T).astype(np.float16)
    assert np.array_equal(got.view(np.float16), want)
    assert np.array_equal(got, O.gemm_q4(X, p, s.view(np.uint16)))


@pytest.mark.parametrize("tile", [3, 4, 12, 14, 15])
def test_q4_gemm_unit_rows_pick_weight_columns(queue, tile):
    # x rows are unit vectors: out[i, :] must be fp16(q * s) of column k_i (nibble order, block of the scale)
    M, N, K = 64, 320, 896
    p, s = mil.quantize_q4(synth_w(1910, N, K))
    ks = (np.arange(M) * 37 + 5) % K
    X = np.zeros((M, K), np.float16)
    X[np.arange(M), ks] = 1.0
    got = _gemm(queue, M, N, K, X, p, s, "q4", tile).view(np.float16)
    want = (_q4_values(p)[:, ks].T.astype(np.float32) * s.astype(np.float32)[:, ks // 32].T).astype(np.float16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("tile", [4, 11, 12, 13, 14, 15])
def test_q4_gemm_repeats_identically(queue, tile):
    M, N, K = 100, 1000, 1024
    print(f"q4 repeat tile mode {tile}", flush=True)
    W, X = synth_w(1940, N, K), synth_x(1941, M, K)
    p, s = mil.quantize_q4(W)
    want = O.gemm_q4(X, p, s.view(np.uint16))
    xb, wb, sb = mil.Buffer.from_host(X), mil.Buffer.from_host(p), mil.Buffer.from_host(s)
    assert mil.nnopt_register_q4_weight(wb, sb, N, K)
    outs = [mil.Buffer(M * N * 2) for _ in range(25)]
    mil.lib().mi_set_gemm_mode(tile)
    try:
        for ob in outs:
            assert mil.pytorch_linear(queue, M, N, K, xb, wb, ob)
        queue.finish()
    finally:
        mil.lib().mi_set_gemm_mode(0)
    first = outs[0].read(np.uint16, (M, N))
    assert_tolerance(first.view(np.float16), want.view(np.float16))
    for i, ob in enumerate(outs[1:]):
        assert np.array_equal(ob.read(np.uint16, (M, N)), first), f"launch {i + 1} differs from launch 0"
    mil.nnopt_unregister_weight(wb)


SAMPLED_ROWS = [0, 1, 31, 32, 63, 64, 127, 128, 159, 160, 255, 256, 1000, 1023, 1024, 2046, 2047]


@pytest.mark.parametrize("N,K", [(4864, 896), (896, 4864)])
def test_q4_prefill_size_rows_sampled(queue, N, K):
    """Config 5 at M = 2048 with Q4 weights, both shapes, as bench.py times them (at N = 896 the library
    cuts K into slices: fp32 partial sums and a reduction launch)."""
    M = 2048
    W, X = synth_w(1920 + N, N, K), synth_x(1921 + N, M, K)
    p, s = mil.quantize_q4(W)
    plan = []
    got = _gemm(queue, M, N, K, X, p, s, "q4", plan=plan)
    assert plan[0][0] == 1 and (plan[0][2] > 1) == (N == 896), plan
    for r in SAMPLED_ROWS:
        want = O.gemv_q4(X[r], p, s.view(np.uint16))
        assert _ulp_apart(got[r], want).max() <= 1, f"row {r}"
    X2 = X.copy()
    X2[5] = X[5] * np.float16(2.0)
    got2 = _gemm(queue, M, N, K, X2, p, s, "q4")
    normal = np.abs(got[5].view(np.float16)) >= np.float16(2.0 ** -13)      # (a subnormal fp16 output has fewer bits)
    assert np.array_equal(got2[5].view(np.float16)[normal], (got[5].view(np.float16) * np.float16(2.0))[normal])
    assert np.array_equal(got2[6], got[6])


def test_fp16_prefill_size_rows_sampled(queue):
    """Config 5 at M = 2048 with fp16 weights, both shapes: sampled rows equal the GEMV of that row of
    x to one fp16 step; doubling a row of x doubles its output row exactly and leaves its neighbour alone."""
    for (N, K) in ((4864, 896), (896, 4864)):
        M = 2048
        W, X = synth_w(2920 + N, N, K), synth_x(2921 + N, M, K)
        got = _gemm(queue, M, N, K, X, W, None, "f16")
        for r in SAMPLED_ROWS:
            want = O.gemv_f16(X[r], W)
            assert _ulp_apart(got[r], want).max() <= 1, f"N={N} K={K} row {r}"
        X2 = X.copy()
        X2[5] = X[5] * np.float16(2.0)
        got2 = _gemm(queue, M, N, K, X2, W, None, "f16")
        normal = np.abs(got[5].view(np.float16)) >= np.float16(2.0 ** -13)      # (a subnormal fp16 output has fewer bits)
        assert np.array_equal(got2[5].view(np.float16)[normal], (got[5].view(np.float16) * np.float16(2.0))[normal])
        assert np.array_equal(got2[6], got[6])


@pytest.mark.parametrize("N,K", [(4864, 896), (896, 4864)])
def test_prefill_size_rows_sampled(queue, N, K):
    """Config 5 at M = 2048, both shapes, the kernels bench.py times: every sampled row of out equals the
    GEMV of that row of x.  At N = 896 the tiles are too few for the chip, so the library cuts K into
    slices (fp32 partial sums in the stream's workspace, then the reduction launch): asserted."""
    M = 2048
    W, X = synth_w(920 + N, N, K), synth_x(921 + N, M, K)
    q, s = mil.quantize_int8(W)
    plan = []
    got = _gemm(queue, M, N, K, X, q, s, "i8", plan=plan)
    assert plan[0][0] == 1 and (plan[0][2] > 1) == (N == 896), plan
    for r in SAMPLED_ROWS:
        want = O.gemv_i8(X[r], q, s.view(np.uint16))
        assert _ulp_apart(got[r], want).max() <= 1, f"row {r}"
    # linearity in x: scaling a row of x by 2 scales the output row by 2 exactly
    X2 = X.copy()
    X2[5] = X[5] * np.float16(2.0)
    got2 = _gemm(queue, M, N, K, X2, q, s, "i8")
    normal = np.abs(got[5].view(np.float16)) >= np.float16(2.0 ** -13)
    assert np.array_equal(got2[5].view(np.float16)[normal], (got[5].view(np.float16) * np.float16(2.0))[normal])
    assert np.array_equal(got2[6], got[6])
    # every row, not only the sampled ones, against the rows-of-GEMV mode of the same entry point
    rows = _gemm(queue, M, N, K, X, q, s, "i8", tile=1)
    assert _ulp_apart(got, rows).max() <= 1
    assert np.mean(got == rows) > 0.99


def test_batched_gemv_mode_stays_bit_exact(queue):
    M, N, K = 32, 896, 896
    W, X = synth_w(930, N, K), synth_x(931, M, K)
    q, s = mil.quantize_int8(W)
    got = _gemm(queue, M, N, K, X, q, s, "i8", tile=1)
    assert np.array_equal(got, O.gemm_i8(X, q, s.view(np.uint16)))


def _random_shapes(seed, count):
    rng = np.random.default_rng(seed)
    shapes = [(2, 1, 64), (3, 7, 64), (16, 33, 128), (17, 255, 192), (31, 257, 64), (33, 1, 1024), (2, 300, 4864)]
    while len(shapes) < count:
        M = int(rng.choice([2, 3, 5, 15, 16, 17, 31, 32, 33, 63, 64, 65, 96, 127, 160, 161, 255, 300]))
        N = int(rng.integers(1, 700))
        K = 64 * int(rng.integers(1, 24))
        shapes.append((M, N, K))
    return shapes


@pytest.mark.parametrize("kind", ["i8", "q4", "f16"])
def test_gemm_random_shapes(queue, kind):
    """Seeded shapes with ragged M and N (one row, one column, one more than a tile, ...), the
    library's own choice of kernel and the wide kernel forced: within one fp16 step of the rows of GEMV."""
    for i, (M, N, K) in enumerate(_random_shapes(77, 36)):
        W, X = synth_w(3000 + i, N, K), synth_x(3100 + i, M, K)
        for tile in (0, 3):
            print(f"{kind} gemm M={M} N={N} K={K} mode {tile}", flush=True)
            if kind == "i8":
                q, s = mil.quantize_int8(W)
                got, want = _gemm(queue, M, N, K, X, q, s, "i8", tile), O.gemm_i8(X, q, s.view(np.uint16))
            elif kind == "q4":
                p, s = mil.quantize_q4(W)
                got, want = _gemm(queue, M, N, K, X, p, s, "q4", tile), O.gemm_q4(X, p, s.view(np.uint16))
            else:
                got, want = _gemm(queue, M, N, K, X, W, None, "f16", tile), O.gemm_f16(X, W)
            assert_tolerance(got.view(np.float16), want.view(np.float16))
            if not (kind == "q4" and tile == 0):
                assert _ulp_apart(got, want).max() <= 1, (M, N, K, tile)


def test_modes_belong_to_the_stream_that_set_them(queue):
    """mi_stream_set_modes: a stream's own gemm / gemv mode holds whatever the process default says,
    and another stream keeps following the default."""
    L = mil.lib()
    M, N, K = 64, 896, 896
    W, X = synth_w(4100, N, K), synth_x(4101, M, K)
    q, s = mil.quantize_int8(W)
    xb, wb, sb = mil.Buffer.from_host(X), mil.Buffer.from_host(q), mil.Buffer.from_host(s)
    assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    other = mil.Queue()
    try:
        assert mil.linear_plan(queue, M, N, K, xb, wb)[0] > 0 and mil.linear_plan(other, M, N, K, xb, wb)[0] > 0
        assert L.mi_stream_set_modes(other.handle, -1, 1) == 1          # rows of GEMV on `other` only
        assert mil.linear_plan(other, M, N, K, xb, wb)[0] == 0
        assert mil.linear_plan(queue, M, N, K, xb, wb)[0] > 0
        a, b = mil.Buffer(M * N * 2), mil.Buffer(M * N * 2)
        assert mil.pytorch_linear(other, M, N, K, xb, wb, a)
        other.finish()
        assert np.array_equal(a.read(np.uint16, (M, N)), O.gemm_i8(X, q, s.view(np.uint16)))   # bit-exact rows
        L.mi_set_gemm_mode(1)                                            # the default changes ...
        assert L.mi_stream_set_modes(other.handle, -1, 3) == 1           # ... `other` pins the wide kernel
        assert mil.linear_plan(queue, M, N, K, xb, wb)[0] == 0
        assert mil.linear_plan(other, M, N, K, xb, wb)[0] == 1
        assert L.mi_stream_set_modes(other.handle, -1, -1) == 1          # forget: back to the default
        assert mil.linear_plan(other, M, N, K, xb, wb)[0] == 0
        assert L.mi_stream_set_modes(other.handle, 5, 0) == 0            # no such gemv mode
    finally:
        L.mi_set_gemm_mode(0)
        L.mi_stream_set_modes(other.handle, -1, -1)
        mil.nnopt_unregister_weight(wb)


# (N, K) of the projections of the three model families the reference ships (stacked q | k | v and
# gate | up as a prompt runs them), and rows of x from a few tokens to a long prompt
_MODEL_PROJECTIONS = [(1152, 896), (896, 896), (9728, 896), (896, 4864),              # Qwen2.5-0.5B
                      (960, 576), (576, 576), (3072, 576), (576, 1536),               # SmolLM2-135M
                      (1536, 1024), (1024, 1024), (9216, 1024), (1024, 4608),         # LFM2-350M
                      (2560, 1024), (8192, 2048)]
_PROMPT_ROWS = [24, 48, 96, 192, 384, 640, 1024, 1536, 2048, 4096]


@pytest.mark.parametrize("kind", ["i8", "f16", "q4"])
def test_planned_kernels_at_model_shapes(queue, kind):
    """The library's own choice of kernel, tile height and K slices (mode 0) at the shapes its fitted
    time estimates were tuned on, two prompt lengths per projection: every element against the
    rows-of-GEMV mode of the same entry point, which the GEMV tests hold to the oracle bit for bit
    (int8, fp16) or within the stated tolerance (Q4)."""
    seen = set()
    for i, (N, K) in enumerate(_MODEL_PROJECTIONS):
        W = synth_w(5000 + i, N, K)
        if kind == "i8":
            w_host, s_host = mil.quantize_int8(W)
        elif kind == "q4":
            w_host, s_host = mil.quantize_q4(W)
        else:
            w_host, s_host = W, None
        for j in range(2):
            M = _PROMPT_ROWS[(3 * i + 5 * j + len(kind)) % len(_PROMPT_ROWS)]
            if M * N > 12_000_000:                          # (bounds the rows-of-GEMV launch)
                M = 256
            X = synth_x(5100 + 2 * i + j, M, K)
            plan = []
            got = _gemm(queue, M, N, K, X, w_host, s_host, kind, plan=plan)
            print(f"{kind} M={M} N={N} K={K} plan {plan[0]}", flush=True)
            seen.add(plan[0][0])
            rows = _gemm(queue, M, N, K, X, w_host, s_host, kind, tile=1)
            assert_tolerance(got.view(np.float16), rows.view(np.float16))
            if kind != "q4":
                assert _ulp_apart(got, rows).max() <= 1, (M, N, K, plan[0])
                assert np.mean(got == rows) > 0.99, (M, N, K, plan[0])
    assert 1 in seen and len(seen) >= 2, seen               # the wide tiles and at least one other kernel ran
