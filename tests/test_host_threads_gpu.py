"""Host threads and streams at the boundary, on the GPU.

The reference's host is single threaded by construction (QW/src/utils.cpp:63-66: plain statics, no
locks).  This library says that several host threads may drive different streams; what that rests on is
checked here: threads that arrive together at the library's first call initialise it once, and a
recorded graph replays on the stream it was recorded on and is refused on any other."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as O
from helpers import ROOT, mil, synth_w, synth_x

pytestmark = pytest.mark.gpu

PROGRAM = r'''
#include "mi_linear.h"
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
/* Four threads whose first library call is mi_stream_create, released together by a barrier; each
 * then runs the same fp16 GEMV on its own stream.  No mi_init call anywhere. */
enum { THREADS = 4, N = 64, K = 256 };
static pthread_barrier_t gate;
static uint16_t W[N * K], x[K], y[THREADS][N];
static int status[THREADS];
static void* work(void* arg) {
    int t = (int)(size_t)arg;
    pthread_barrier_wait(&gate);
    void* s = mi_stream_create();
    if (!s) { status[t] = 1; return 0; }
    void* Wd = mi_malloc(sizeof W);
    void* xd = mi_malloc(sizeof x);
    void* yd = mi_malloc(N * 2);
    if (!Wd || !xd || !yd) { status[t] = 2; return 0; }
    if (!mi_memcpy_h2d(Wd, W, sizeof W, s) || !mi_memcpy_h2d(xd, x, sizeof x, s)) { status[t] = 3; return 0; }
    for (int rep = 0; rep < 50; ++rep)
        if (!mi_linear(s, 1, N, K, xd, Wd, yd)) { status[t] = 4; return 0; }
    if (!mi_memcpy_d2h(y[t], yd, N * 2, s)) { status[t] = 5; return 0; }
    mi_free(Wd); mi_free(xd); mi_free(yd);
    if (!mi_stream_destroy(s)) status[t] = 6;
    return 0;
}
int main(void) {
    mi_synth_normal_f16(41, 0.02, N * K, W);
    mi_synth_normal_f16(42, 1.0, K, x);
    pthread_barrier_init(&gate, 0, THREADS);
    pthread_t th[THREADS];
    for (size_t t = 0; t < THREADS; ++t) pthread_create(&th[t], 0, work, (void*)t);
    for (int t = 0; t < THREADS; ++t) pthread_join(th[t], 0);
    for (int t = 0; t < THREADS; ++t) {
        if (status[t]) { printf("thread %d failed at %d\n", t, status[t]); return 1; }
        if (memcmp(y[t], y[0], sizeof y[0])) { printf("thread %d differs\n", t); return 1; }
    }
    printf("%s %d", mi_device_arch(), mi_device_cus());
    for (int n = 0; n < N; ++n) printf(" %u", (unsigned)y[0][n]);
    printf("\n");
    return 0;
}
'''


def test_threads_that_arrive_together_at_the_first_call(tmp_path):
    src = tmp_path / "first.c"
    src.write_text(PROGRAM)
    exe = tmp_path / "first"
    libdir = os.path.dirname(mil.LIB_PATH)
    subprocess.check_call(["gcc", "-std=gnu11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src),
                           "-o", str(exe), "-L", libdir, "-lmi_linear", f"-Wl,-rpath,{libdir}", "-lpthread"])
    print("four threads, first call mi_stream_create", flush=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.stdout, r.stderr[-2000:])
    fields = r.stdout.split()
    assert fields[0].startswith("gfx950") and int(fields[1]) > 0
    W, x = synth_w(41, 64, 256), synth_x(42, 256)
    assert np.array_equal(np.array(fields[2:], np.uint16), O.gemv_f16(x, W))


def test_graph_replays_on_its_recording_stream_only(capfd):
    assert mil.lib().mi_init(0) == 1
    qa, qb = mil.Queue(), mil.Queue()
    N, K = 896, 4864
    W, x = synth_w(51, N, K), synth_x(52, K)
    q, s = mil.quantize_int8(W)
    Wb, sb, xb, ob = mil.Buffer.from_host(q), mil.Buffer.from_host(s), mil.Buffer.from_host(x), mil.Buffer(N * 2)
    assert mil.nnopt_register_int8_weight(Wb, sb, N, K)
    assert mil.pytorch_linear(qa, 1, N, K, xb, Wb, ob)          # loads the kernel's code before the recording
    qa.finish()
    with mil.Graph(qa) as g:
        assert mil.pytorch_linear(qa, 1, N, K, xb, Wb, ob)
    ob.write(np.zeros(N, np.uint16))
    capfd.readouterr()
    with pytest.raises(RuntimeError):
        g.launch(qb)
    assert "recorded on stream" in capfd.readouterr().err
    qb.finish()
    assert not ob.read(np.uint16, (N,)).any()                    # nothing ran
    with pytest.raises(RuntimeError):
        g.launch(mil.Queue(default=True))
    g.launch()
    qa.finish()
    assert np.array_equal(ob.read(np.uint16, (N,)), O.gemv_i8(x, q, s.view(np.uint16)))
    mil.nnopt_unregister_weight(Wb)
