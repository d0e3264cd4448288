"""Throughput variant of the Q4 GEMV (mi_set_gemv_mode(1), the default): same fp32 products as
the reference kernel, summed in another order.  Bar: the stated tolerance (max-abs/rel 1e-3,
cosine >= 0.9999) against the oracle, bit-exact wherever the arithmetic is exact (integer
data, unit vectors), and bit-exact unpack indexing over all byte values."""
import numpy as np
import pytest

import oracle_lib as O
from helpers import assert_tolerance, mil, synth_w, synth_x

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def queue():
    assert mil.lib().mi_init(0) == 1, "no gfx950 device"
    mil.lib().mi_set_gemv_mode(1)
    q = mil.Queue()
    yield q
    q.finish()


def _run(queue, N, K, x, p, sc, add_to=None):
    xb, pb, sb = mil.Buffer.from_host(x), mil.Buffer.from_host(p), mil.Buffer.from_host(sc)
    assert mil.nnopt_register_q4_weight(pb, sb, N, K)
    pad = 64
    guard = np.full(N + 2 * pad, 0x7BCD, np.uint16)
    if add_to is not None:
        guard[pad:-pad] = add_to.view(np.uint16)
    ob = mil.Buffer.from_host(guard)
    if add_to is None:
        assert mil.pytorch_linear(queue, 1, N, K, xb, pb, ob.ptr + 2 * pad)
    else:
        assert mil.pytorch_linear_add(queue, 1, N, K, xb, pb, ob.ptr + 2 * pad)
    queue.finish()
    full = ob.read(np.uint16, guard.shape)
    assert np.all(full[:pad] == 0x7BCD) and np.all(full[-pad:] == 0x7BCD)
    mil.nnopt_unregister_weight(pb)
    return full[pad:-pad]


@pytest.mark.parametrize("N,K", [(4864, 896), (151936, 896), (4608, 1024), (8192, 576), (4100, 1536), (4099, 896),
                                 (8192, 2048), (4101, 2048), (4100, 2560), (49152, 960), (4100, 960),
                                 # K values without an instance of their own: the same arithmetic with x in LDS
                                 (4099, 1280), (4096, 3072), (4098, 4096), (4096, 8192), (4097, 11008),
                                 (4096, 32), (4100, 30720)])
def test_fast_q4_within_tolerance(queue, N, K):
    print(f"fast q4 N={N} K={K}", flush=True)
    W, x = synth_w(1000 + N, N, K), synth_x(1100 + K, K)
    p, sc = mil.quantize_q4(W)
    got = _run(queue, N, K, x, p, sc)
    want = O.gemv_q4(x, p, sc.view(np.uint16))
    assert_tolerance(got.view(np.float16), want.view(np.float16))
    same = float(np.mean(got == want))
    print(f"fast q4 N={N} K={K} identical halves {same:.4f}", flush=True)
    # Nearly all outputs are the same half.  The others sit next to a rounding boundary, where another order
    # of the same fp32 additions lands on the other side; a longer row has more additions, and the share grows
    # about as sqrt(K).  Measured: 0.966 at K = 32, 0.987 at 576, 0.972 at 896, 0.956 at 2560, 0.945 at 8192,
    # 0.923 at 11 008.  The line below follows those with a margin of 0.01 to 0.03; an error in how the staged x
    # is paired or ordered moves every output and falls far below it at any K.
    assert same > 0.96 - 0.0005 * np.sqrt(K)


@pytest.mark.parametrize("K", [896, 2048, 2560, 960, 3072, 8192, 11008, 30720])
def test_fast_q4_exact_on_integer_data_and_all_bytes(queue, K):
    # integer activations and power-of-two scales: every order of the fp32 sum is exact
    rng = np.random.default_rng(5)
    N = 4096
    p = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    p[0, :256] = np.arange(256, dtype=np.uint8)
    sc = (2.0 ** rng.integers(-8, -3, (N, K // 32))).astype(np.float16)
    x = rng.integers(-4, 5, K).astype(np.float16)
    got = _run(queue, N, K, x, p, sc)
    nib = np.stack([p & 15, p >> 4], -1).reshape(N, K).astype(np.int64) - 8
    want = ((nib * np.repeat(sc.astype(np.float64), 32, axis=1)) @ x.astype(np.float64)).astype(np.float16)
    assert np.array_equal(got.view(np.float16), want)
    assert np.array_equal(got, O.gemv_q4(x, p, sc.view(np.uint16)))


@pytest.mark.parametrize("K", [896, 1280, 11008])
def test_fast_q4_unit_vectors_and_subnormal_activations(queue, K):
    N = 4096
    W = synth_w(1200, N, K)
    p, sc = mil.quantize_q4(W)
    nib = np.stack([p & 15, p >> 4], -1).reshape(N, K).astype(np.float32) - 8
    for k in (0, 1, 4, 5, 31, 32, 511, 512, 895, K // 2 + 17, K - 33, K - 1):
        x = np.zeros(K, np.float16)
        x[k] = 1.0
        want = (nib[:, k] * sc[:, k // 32].astype(np.float32)).astype(np.float16)
        assert np.array_equal(_run(queue, N, K, x, p, sc).view(np.float16), want), k
    x = synth_x(1201, K)
    x[::5] = np.float16(6e-8)
    x[1::5] = np.float16(-2e-5)
    got = _run(queue, N, K, x, p, sc)
    assert_tolerance(got.view(np.float16), O.gemv_q4(x, p, sc.view(np.uint16)).view(np.float16))


@pytest.mark.parametrize("K", [896, 3072])
def test_fast_q4_residual_epilogue(queue, K):
    N = 8192
    W, x = synth_w(1300, N, K), synth_x(1301, K)
    res0 = synth_x(1302, N)
    p, sc = mil.quantize_q4(W)
    got = _run(queue, N, K, x, p, sc, add_to=res0)
    want = res0.view(np.uint16).copy()
    O.lib.orc_gemv_q4_add(O.u16(x), p, np.ascontiguousarray(sc.view(np.uint16)), want, N, K)
    assert_tolerance(got.view(np.float16), want.view(np.float16))


@pytest.mark.parametrize("K", [896, 3072])
def test_fast_q4_rows_of_a_small_batch_equal_single_calls(queue, K):
    """Three rows of x in one call (each row a GEMV of its own, gemm mode 1) and the same rows one
    call each: the same kernel either way, so the same bits; K with an instance of its own and K
    through the kernel that keeps x in LDS."""
    N, M = 4100, 3
    W, X = synth_w(1400 + K, N, K), synth_x(1401 + K, M, K)
    p, sc = mil.quantize_q4(W)
    singles = np.stack([_run(queue, N, K, X[i], p, sc) for i in range(M)])
    xb, pb, sb = mil.Buffer.from_host(X), mil.Buffer.from_host(p), mil.Buffer.from_host(sc)
    ob = mil.Buffer(M * N * 2)
    assert mil.nnopt_register_q4_weight(pb, sb, N, K)
    mil.lib().mi_set_gemm_mode(1)
    try:
        assert mil.pytorch_linear(queue, M, N, K, xb, pb, ob)
        queue.finish()
    finally:
        mil.lib().mi_set_gemm_mode(0)
        mil.nnopt_unregister_weight(pb)
    got = ob.read(np.uint16, (M, N))
    assert np.array_equal(got, singles)
    for i in range(M):
        assert_tolerance(got[i].view(np.float16), O.gemv_q4(X[i], p, sc.view(np.uint16)).view(np.float16))
