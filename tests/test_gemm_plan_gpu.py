"""The GEMM planner against the kernels it chooses among, by the clock.

Which kernel, tile height and number of K slices `pytorch_linear` runs for M > 1 comes from time estimates
fitted to measurements on one MI355X (plan_gemm).  The parity tests hold every plan to the oracle; this one
holds the choice to the clock, so that a compiler or runtime update that shifts the kernels' relative speed
shows up as a failure instead of a silent slowdown: at the projections of the three model families and three
prompt lengths, the library's own choice (mode 0) must not be more than 25 % behind the fastest pinned kernel
(mi_set_gemm_mode 2, 3, 5, 11..15).  Contract of the call: QW/src/utils.cpp:785-796."""
import numpy as np
import pytest

from helpers import mil, synth_w, synth_x

pytestmark = pytest.mark.gpu

# (N, K): q|k|v stacked, o, gate|up stacked, down of Qwen2.5-0.5B; SmolLM2-135M; LFM2-350M
SHAPES = [(1152, 896), (896, 896), (9728, 896), (896, 4864),
          (960, 576), (576, 576), (3072, 576), (576, 1536),
          (1536, 1024), (1024, 1024), (9216, 1024), (1024, 4608)]
ROWS = [64, 512, 2048]
CALLS, REPLAYS = 8, 7
BEHIND = 1.25


@pytest.fixture(scope="module")
def queue():
    assert mil.lib().mi_init(0) == 1, "no gfx950 device"
    q = mil.Queue()
    yield q
    q.finish()
    mil.lib().mi_set_gemm_mode(0)


def _time_us(queue, mode, M, N, K, xb, wb, ob):
    """Median over REPLAYS graph replays of CALLS calls, per call; None where the mode has no kernel."""
    mil.lib().mi_set_gemm_mode(mode)
    try:
        kern, rows, slices = mil.linear_plan(queue, M, N, K, xb, wb)
        if kern < 0:
            return None, None
        arr = mil.make_calls([(M, N, K, xb, wb, ob)] * CALLS)
        assert mil.linear_batch(queue, arr) == CALLS          # loads the code before the recording
        queue.finish()
        with mil.Graph(queue) as g:
            assert mil.linear_batch(queue, arr) == CALLS
        g.launch()
        queue.finish()
        e0, e1 = mil.Event(), mil.Event()
        got = []
        for _ in range(REPLAYS):
            e0.record(queue)
            g.launch()
            e1.record(queue)
            e1.synchronize()
            got.append(e0.elapsed_ms(e1) * 1e3 / CALLS)
        got.sort()
        return got[len(got) // 2], (kern, rows, slices)
    finally:
        mil.lib().mi_set_gemm_mode(0)


@pytest.mark.parametrize("N,K", SHAPES)
def test_the_planners_choice_is_near_the_fastest_pinned_kernel(queue, N, K):
    q, s = mil.quantize_int8(synth_w(7000 + N, N, K))
    wb, sb = mil.Buffer.from_host(q), mil.Buffer.from_host(s)
    assert mil.nnopt_register_int8_weight(wb, sb, N, K)
    try:
        for M in ROWS:
            xb, ob = mil.Buffer.from_host(synth_x(7100 + M, M, K)), mil.Buffer(M * N * 2)
            modes = [2, 3] + [10 + t for t in range(1, 6) if 32 * (t - 1) < M] + ([5] if M <= 64 else [])
            worst = None
            for attempt in range(3):                    # further looks before a failure: boxes jitter
                own, plan = _time_us(queue, 0, M, N, K, xb, wb, ob)
                pinned = {}
                for mode in modes:
                    us, _ = _time_us(queue, mode, M, N, K, xb, wb, ob)
                    if us is not None:
                        pinned[mode] = us
                best_mode = min(pinned, key=pinned.get)
                print(f"int8 M={M} N={N} K={K} plan {plan} own {own:.2f} us, best pinned: mode {best_mode} "
                      f"{pinned[best_mode]:.2f} us", flush=True)
                worst = (own, best_mode, pinned[best_mode], plan)
                if own <= BEHIND * pinned[best_mode]:
                    worst = None
                    break
            assert worst is None, f"M={M} N={N} K={K}: chose {worst[3]} at {worst[0]:.2f} us, mode {worst[1]} takes {worst[2]:.2f} us"
    finally:
        mil.nnopt_unregister_weight(wb)
