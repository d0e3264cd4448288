"""Greedy-token argmax: the oracle's literal restatement of the reference's two kernels
(QW/kernels/gemv_m1.cl:198-280) against an independent statement of the tie order they imply, and
the one-launch device kernel against the oracle, through the C ABI."""
import numpy as np
import pytest

import oracle_lib as O
from helpers import mil

NEG_INF = np.float16(-np.inf)


def tie_order_argmax(x, num_partials):
    """What the two kernels compute, said differently.  Work-item t scans t, t + 64, ... with a
    strict ">" (first maximum wins), then a tree merges position t + s into t for s = 32 .. 1,
    again with a strict ">": two equal maxima meet at the lowest bit in which their work-item
    numbers differ and the one with a 0 there stays, i.e. the smaller BIT-REVERSED work-item
    number wins.  So among the candidates (values > -FLT_MAX: neither NaN nor -inf) with the
    greatest value the winner has the chunk p with the lowest (bitrev6(p % 64), p), then the lowest
    bitrev6((i - chunk start) % 64), then the lowest i; 0 with no candidate."""
    v = np.asarray(x, np.float16).astype(np.float32)
    n = v.size
    chunk = (n + num_partials - 1) // num_partials
    ok = v > np.float32(-3.402823466e+38)          # False for NaN and -inf
    if not ok.any():
        return 0
    top = v[ok].max()
    idx = np.nonzero(ok & (v == top))[0]
    def bitrev6(a):
        r = np.zeros_like(a)
        for b in range(6):
            r |= ((a >> b) & 1) << (5 - b)
        return r
    p = idx // chunk
    lane = (idx - p * chunk) % 64
    order = np.lexsort((idx, bitrev6(lane), p, bitrev6(p % 64)))      # last key is the primary one
    return int(idx[order[0]])


def cases():
    rng = np.random.default_rng(11)
    out = []
    for n in (1, 7, 63, 64, 65, 1000, 4097, 151936):
        out.append((f"normal{n}", rng.standard_normal(n).astype(np.float16)))
    # few distinct values: many equal maxima spread over chunks and lanes
    for n in (130, 5000, 151936):
        out.append((f"ties{n}", rng.integers(-3, 4, n).astype(np.float16)))
    x = np.full(151936, -2.0, np.float16)
    x[[150000, 70, 4748 * 3 + 5, 4748 * 3 + 64 + 2, 9]] = 1.5      # same value in several chunks and lanes
    out.append(("planted", x))
    x = np.full(9000, NEG_INF)
    out.append(("all-inf", x))
    x = rng.standard_normal(9000).astype(np.float16)
    x[::3] = np.float16(np.nan)
    x[5] = np.float16(np.inf)
    x[4000] = np.float16(np.inf)
    out.append(("nan-and-inf", x))
    out.append(("all-nan", np.full(300, np.float16(np.nan))))
    return out


@pytest.mark.parametrize("name,x", cases(), ids=[c[0] for c in cases()])
@pytest.mark.parametrize("num_partials", [1, 32, 64, 100, 257])
def test_oracle_argmax_follows_the_kernels_tie_order(name, x, num_partials):
    assert O.argmax_f16(x, num_partials) == tie_order_argmax(x, num_partials)


def test_oracle_argmax_plain_cases():
    x = np.zeros(151936, np.float16)
    x[123456] = 3.0
    assert O.argmax_f16(x) == 123456
    # a tie inside one chunk: index 66 (work-item 2 = 000010b) beats index 5 (work-item 5 = 000101b),
    # they differ first in bit 0 and 2 has a 0 there
    x = np.zeros(4096, np.float16)
    x[[5, 66]] = 1.0
    assert O.argmax_f16(x, 1) == 66
    assert O.argmax_f16(x, 4096 // 64) == 5        # chunks of 64: index 5 sits in chunk 0, 66 in chunk 1
    # work-item 34 (100010b) beats work-item 3 (000011b): bit 0 decides
    x = np.zeros(64, np.float16)
    x[[3, 34]] = 1.0
    assert O.argmax_f16(x, 1) == 34


def test_chunk_index_by_reciprocal_multiply_is_exact():
    """The device tie rule finds an index's chunk as trunc(double(i) * (1.0 / chunk)), corrected by
    one where the remainder i - q * chunk falls outside [0, chunk) (argmax_rule.h, chunk_of).  The
    same IEEE double operations in numpy: equal to i // chunk for every index below 2^31, at the
    chunk boundaries where a rounded reciprocal could land on the wrong side."""
    rng = np.random.default_rng(3)
    chunks = np.unique(np.concatenate([
        np.array([1, 2, 3, 5, 7, 10, 63, 64, 65, 592, 1520, 4748, 151936, 2**20, 2**30, 2**31 - 1]),
        rng.integers(1, 2**31 - 1, 2000), rng.integers(1, 70000, 2000)])).astype(np.int64)
    top = np.int64(2**31 - 1)
    for c in chunks:
        k = np.unique(np.concatenate([np.arange(0, 40), rng.integers(0, top // c + 1, 300), [top // c]])).astype(np.int64)
        idx = np.unique(np.clip(np.concatenate([k * c - 1, k * c, k * c + 1, [top]]), 0, top))
        inv = np.float64(1.0) / np.float64(c)
        q = np.trunc(idx.astype(np.float64) * inv).astype(np.int64)
        r = idx - q * c
        assert np.all((r >= -c) & (r < 2 * c)), int(c)           # off by one at most
        q = q + np.where(r < 0, -1, np.where(r >= c, 1, 0))
        assert np.array_equal(q, idx // c), int(c)


@pytest.mark.gpu
@pytest.mark.parametrize("name,x", cases(), ids=[c[0] for c in cases()])
def test_device_argmax_matches_oracle(name, x):
    assert mil.lib().mi_init(0) == 1
    q = mil.Queue()
    tok = mil.Buffer.from_host(np.array([-7], np.int32))
    for num_partials in (32, 1, 100):
        for shift in (0, 1):                       # also a logits pointer that is not 16-byte aligned
            host = np.concatenate([np.zeros(shift, np.float16), x])
            xb = mil.Buffer.from_host(host)
            assert mil.argmax_f16(q, xb.ptr + 2 * shift, x.size, tok, num_partials)
            q.finish()
            got = int(tok.read(np.int32, (1,))[0])
            assert got == O.argmax_f16(x, num_partials), (name, num_partials, shift)


@pytest.mark.gpu
def test_lm_head_then_argmax_on_device():
    """mi_linear_argmax: logits as mi_linear writes them, token as the oracle picks it from them."""
    from helpers import synth_w, synth_x
    assert mil.lib().mi_init(0) == 1
    q = mil.Queue()
    mil.lib().mi_set_gemv_mode(0)
    try:
        N, K = 20000, 896
        W, x = synth_w(51, N, K), synth_x(52, 1, K).reshape(K)
        W[[17, 9000, 19999]] = W[4242]             # identical rows: identical logits, a real tie if they are the top
        qw, s = mil.quantize_int8(W)
        wb, sb, xb = mil.Buffer.from_host(qw), mil.Buffer.from_host(s), mil.Buffer.from_host(x)
        assert mil.nnopt_register_int8_weight(wb, sb, N, K)
        logits, tok = mil.Buffer(N * 2), mil.Buffer.from_host(np.array([-1], np.int32))
        assert mil.pytorch_linear_argmax(q, N, K, xb, wb, logits, tok)
        q.finish()
        want_logits = O.gemv_i8(x, qw, s.view(np.uint16))
        assert np.array_equal(logits.read(np.uint16, (N,)), want_logits)
        assert int(tok.read(np.int32, (1,))[0]) == O.argmax_f16(want_logits)
        # make the tied rows the winners: scale x so that row 4242's logit is the top by construction
        best = int(np.argmax(want_logits.view(np.float16).astype(np.float32)))
        W2 = W.copy()
        W2[[17, 9000, 19999, 4242]] = W[best]
        qw2, s2 = mil.quantize_int8(W2)
        wb2, sb2 = mil.Buffer.from_host(qw2), mil.Buffer.from_host(s2)
        assert mil.nnopt_register_int8_weight(wb2, sb2, N, K)
        assert mil.pytorch_linear_argmax(q, N, K, xb, wb2, logits, tok)
        q.finish()
        want2 = O.gemv_i8(x, qw2, s2.view(np.uint16))
        assert np.array_equal(logits.read(np.uint16, (N,)), want2)
        v = want2.view(np.float16).astype(np.float32)
        tied = np.nonzero(v == v.max())[0]
        assert tied.size >= 5, tied                 # the tie is real
        assert int(tok.read(np.int32, (1,))[0]) == O.argmax_f16(want2), tied
        mil.nnopt_unregister_weight(wb)
        mil.nnopt_unregister_weight(wb2)
    finally:
        mil.lib().mi_set_gemv_mode(1)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,N,K", [("int8", 151936, 896), ("fp16", 151936, 896), ("int8", 49152, 576),
                                      ("fp16", 30001, 1536), ("int8", 5000, 4864), ("int8", 300, 1024),
                                      ("q4", 20000, 896), ("q4", 151936, 896), ("q4", 5000, 576), ("q4", 3000, 1024),
                                      ("int8", 7000, 640)])
def test_argmax_inside_the_lm_head_launch(kind, N, K):
    """Where the GEMV keeps x in registers (int8 and fp16 at the K of the model families, Q4 where its
    throughput kernel runs) its wavefronts leave their best rows and a small launch picks the token
    from those; other K, and Q4 launches too small for that kernel, read the logits back.  Either way: logits as mi_linear's, token as the oracle's from those logits, with
    thousands of equal maxima (W has 40 distinct rows) and for several chunkings."""
    from helpers import synth_w, synth_x
    assert mil.lib().mi_init(0) == 1
    q = mil.Queue()
    rng = np.random.default_rng(N + K)
    rows = synth_w(71, 40, K)
    W = rows[rng.integers(0, 40, N)]
    x = synth_x(72, 1, K).reshape(K)
    xb = mil.Buffer.from_host(x)
    if kind == "int8":
        qw, s = mil.quantize_int8(W)
        wb, sb = mil.Buffer.from_host(qw), mil.Buffer.from_host(s)
        assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    elif kind == "q4":
        qw, s = mil.quantize_q4(W)
        wb, sb = mil.Buffer.from_host(qw), mil.Buffer.from_host(s)
        assert mil.nnopt_register_q4_weight(wb, sb, N, K)
    else:
        wb = mil.Buffer.from_host(W)
    plain, logits = mil.Buffer(N * 2), mil.Buffer(N * 2)
    tok = mil.Buffer.from_host(np.array([-1], np.int32))
    try:
        assert mil.pytorch_linear(q, 1, N, K, xb, wb, plain)
        q.finish()
        want_logits = plain.read(np.uint16, (N,))
        v = want_logits.view(np.float16).astype(np.float32)
        assert (v == v.max()).sum() >= max(2, min(20, N // 300))
        for num_partials in (32, 1, 100, 257):
            tok.write(np.array([-1], np.int32))
            assert mil.pytorch_linear_argmax(q, N, K, xb, wb, logits, tok, num_partials)
            q.finish()
            assert np.array_equal(logits.read(np.uint16, (N,)), want_logits)
            assert int(tok.read(np.int32, (1,))[0]) == O.argmax_f16(want_logits, num_partials), num_partials
        # logits that are no candidates (x = -inf gives NaN and -inf only): token 0
        xb2 = mil.Buffer.from_host(np.full(K, -np.inf, np.float16))
        assert mil.pytorch_linear_argmax(q, N, K, xb2, wb, logits, tok)
        q.finish()
        got = logits.read(np.uint16, (N,))
        assert int(tok.read(np.int32, (1,))[0]) == O.argmax_f16(got)
    finally:
        if kind != "fp16":
            mil.nnopt_unregister_weight(wb)


@pytest.mark.gpu
def test_stream_without_workspace_takes_the_one_launch_paths():
    """A hipStream_t that mi_stream_create did not make has no workspace: the argmax runs as one
    block and an int8 GEMM that would cut K into slices runs unsliced.  Same results."""
    import ctypes
    from helpers import synth_w, synth_x
    assert mil.lib().mi_init(0) == 1
    hip = ctypes.CDLL("libamdhip64.so")
    foreign = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(foreign)) == 0
    try:
        own = mil.Queue()
        x = np.random.default_rng(5).integers(-3, 4, 151936).astype(np.float16)     # thousands of ties
        xb = mil.Buffer.from_host(x)
        t_own, t_foreign = mil.Buffer.from_host(np.array([-1], np.int32)), mil.Buffer.from_host(np.array([-1], np.int32))
        assert mil.argmax_f16(own, xb, x.size, t_own)
        assert mil.lib().mi_argmax_f16(foreign, xb.ptr, x.size, 32, t_foreign.ptr)
        own.finish()
        assert hip.hipStreamSynchronize(foreign) == 0
        want = O.argmax_f16(x)
        assert int(t_own.read(np.int32, (1,))[0]) == want
        assert int(t_foreign.read(np.int32, (1,))[0]) == want
        # GEMM: 64 x 896 x 4864 is a shape the library slices along K when it has a workspace
        M, N, K = 64, 896, 4864
        W, X = synth_w(61, N, K), synth_x(62, M, K)
        qw, s = mil.quantize_int8(W)
        wb, sb, Xb = mil.Buffer.from_host(qw), mil.Buffer.from_host(s), mil.Buffer.from_host(X)
        assert mil.nnopt_register_int8_weight(wb, sb, N, K)
        o_own, o_foreign = mil.Buffer(M * N * 2), mil.Buffer(M * N * 2)
        assert mil.pytorch_linear(own, M, N, K, Xb, wb, o_own)
        assert mil.lib().mi_linear(foreign, M, N, K, Xb.ptr, wb.ptr, o_foreign.ptr)
        own.finish()
        assert hip.hipStreamSynchronize(foreign) == 0
        want = O.gemm_i8(X, qw, s.view(np.uint16)).view(np.float16)
        from helpers import assert_tolerance
        assert_tolerance(o_own.read(np.float16, (M, N)), want)
        assert_tolerance(o_foreign.read(np.float16, (M, N)), want)
        mil.nnopt_unregister_weight(wb)
    finally:
        hip.hipStreamDestroy(foreign)
