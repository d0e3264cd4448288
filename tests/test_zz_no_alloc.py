"""mi_linear_argmax_static, the entry point that allocates nothing (its kernels' scratch is an
array inside the library's code object): same logits and token as mi_linear_argmax on the same
inputs, bit for bit, on two calls in a row of which the second is smaller, so that anything the
first call left in the shared scratch would show; on a stream the library did not create (which
has no workspace of its own); for a weight kind and K that take the two-launch argmax; and the
refusal of a size beyond the stated maximum."""
import ctypes

import numpy as np
import pytest

import oracle_lib as O
from helpers import mil, synth_w, synth_x


def _case(kind, N, K, seed):
    rng = np.random.default_rng(seed)
    rows = synth_w(seed, 40, K)
    W = rows[rng.integers(0, 40, N)]            # 40 distinct rows: thousands of tied logits
    x = synth_x(seed + 1, 1, K).reshape(K)
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
        wb, sb = mil.Buffer.from_host(W), None
    return dict(kind=kind, N=N, K=K, x=xb, W=wb, S=sb)


def _both(own, stream_handle, sync, c, num_partials):
    """(logits, token) of the existing entry point on the library's stream and of the static one on stream_handle."""
    N, K = c["N"], c["K"]
    la, lb = mil.Buffer(N * 2), mil.Buffer(N * 2)
    ta, tb = mil.Buffer.from_host(np.array([-1], np.int32)), mil.Buffer.from_host(np.array([-2], np.int32))
    assert mil.pytorch_linear_argmax(own, N, K, c["x"], c["W"], la, ta, num_partials)
    own.finish()
    assert mil.lib().mi_linear_argmax_static(stream_handle, N, K, c["x"].ptr, c["W"].ptr, lb.ptr, num_partials, tb.ptr)
    sync()
    return (la.read(np.uint16, (N,)), int(ta.read(np.int32, (1,))[0]),
            lb.read(np.uint16, (N,)), int(tb.read(np.int32, (1,))[0]))


@pytest.mark.gpu
def test_static_scratch_entry_point_matches_the_allocating_one():
    assert mil.lib().mi_init(0) == 1
    hip = ctypes.CDLL("libamdhip64.so")
    foreign = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(foreign)) == 0
    own = mil.Queue()
    cases = []
    try:
        # big then small on the same scratch: the small launch's wavefronts mostly have no rows
        big = _case("int8", 151936, 896, 301)
        small = _case("int8", 300, 896, 302)
        mid = _case("fp16", 30001, 1536, 303)
        q4 = _case("q4", 20000, 896, 304)            # fused argmax in the throughput Q4 kernel
        odd = _case("int8", 7000, 640, 305)          # K the fused path does not take: two-launch argmax
        cases = [big, small, mid, q4, odd]
        for stream_handle, sync in ((foreign, lambda: hip.hipStreamSynchronize(foreign)),
                                    (own.handle, own.finish)):
            for c, parts in ((big, 32), (small, 32), (big, 257), (mid, 1), (small, 100), (q4, 32), (odd, 32),
                             (small, 32)):
                print(f"static argmax: {c['kind']} N={c['N']} K={c['K']} partials={parts}", flush=True)
                la, ta, lb, tb = _both(own, stream_handle, sync, c, parts)
                assert np.array_equal(la, lb), (c["kind"], c["N"])
                assert ta == tb == O.argmax_f16(la, parts), (c["kind"], c["N"], parts, ta, tb)
        # it allocates nothing: every kernel above has run once (its code is loaded), and across further
        # calls of every path, on both streams, the device's free memory does not move
        def free_bytes():
            free, total = ctypes.c_size_t(), ctypes.c_size_t()
            assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
            return free.value
        outs = {id(c): (mil.Buffer(c["N"] * 2), mil.Buffer(4)) for c in cases}
        own.finish()
        hip.hipStreamSynchronize(foreign)
        before = free_bytes()
        for stream_handle, sync in ((foreign, lambda: hip.hipStreamSynchronize(foreign)), (own.handle, own.finish)):
            for c, parts in ((big, 32), (small, 100), (mid, 1), (q4, 32), (odd, 32)):
                lb, tb = outs[id(c)]
                assert mil.lib().mi_linear_argmax_static(stream_handle, c["N"], c["K"], c["x"].ptr, c["W"].ptr, lb.ptr,
                                                         parts, tb.ptr)
                assert free_bytes() == before, (c["kind"], c["N"])
            sync()
            assert free_bytes() == before
        # beyond the stated maximum: refused before anything is launched.  W is plain fp16 memory that
        # no registration describes, so nothing but the limit itself can be what refuses the call.
        too_many = (1 << 22) + 4
        tok = mil.Buffer.from_host(np.array([-7], np.int32))
        plain_w = mil.Buffer(4096)
        assert mil.lib().mi_weight_kind(plain_w.ptr) == 0
        assert mil.lib().mi_linear_argmax_static(own.handle, too_many, 896, big["x"].ptr, plain_w.ptr,
                                                 big["W"].ptr, 32, tok.ptr) == 0
        own.finish()
        assert int(tok.read(np.int32, (1,))[0]) == -7
    finally:
        for c in cases:
            if c["kind"] != "fp16":
                mil.nnopt_unregister_weight(c["W"])
        hip.hipStreamDestroy(foreign)
