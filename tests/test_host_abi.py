"""C-ABI library: loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

from helpers import ROOT, mil


def _declared():
    names = set()
    for header in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert len(names) >= 35
    lib = ctypes.CDLL(mil.LIB_PATH)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_every_declared_symbol():
    assert sorted(mil._SIGNATURES) == _declared()


def test_register_argument_checks_need_no_gpu(capfd):
    L = mil.lib()
    # null / non-positive arguments -> false (LF/src/utils.cpp:358, 585)
    assert L.mi_register_int8_weight(None, 0x1000, 4, 4) == 0
    assert L.mi_register_int8_weight(0x1000, None, 4, 4) == 0
    assert L.mi_register_int8_weight(0x1000, 0x2000, 0, 4) == 0
    assert L.mi_register_q4_weight(0x1000, 0x2000, 4, -1) == 0
    # Q4 with a K that is not a whole number of 32-blocks is refused, as the quantizer does
    assert L.mi_register_q4_weight(0x1000, 0x2000, 4, 48) == 0
    assert "ERROR:" in capfd.readouterr().err
    # registry bookkeeping
    assert L.mi_register_int8_weight(0x1000, 0x2000, 8, 64) == 1
    assert L.mi_weight_kind(0x1000) == 8
    assert L.mi_register_q4_weight(0x1000, 0x2000, 8, 64) == 1       # re-registration overwrites
    assert L.mi_weight_kind(0x1000) == 4
    assert L.mi_unregister_weight(0x1000) == 1
    assert L.mi_weight_kind(0x1000) == 0
    assert L.mi_unregister_weight(0x1000) == 0


def test_headers_are_plain_c_and_a_c_program_links(tmp_path):
    """The boundary is a C ABI: both headers compile as C11 with gcc (no C++, no HIP types), and a C
    program that calls the host-only entry points links against the library and runs without a GPU."""
    import subprocess
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include "mi_linear.h"
#include "mi_decode.h"
#include <stdio.h>
#include <string.h>
int main(void) {
    uint16_t w[2 * 32];
    int8_t q[2 * 32];
    uint8_t p[2 * 16];
    uint16_t s8[2], s4[2];
    mi_synth_normal_f16(7, 0.02, 2 * 32, w);
    if (!mi_quantize_int8(w, 2, 32, q, s8)) return 1;
    if (!mi_quantize_q4(w, 2, 32, p, s4)) return 2;
    mi_linear_call call;
    memset(&call, 0, sizeof call);
    mi_decoder_config cfg;
    memset(&cfg, 0, sizeof cfg);
    if (mi_decoder_create(&cfg, 0) != 0) return 3;          /* refused: bad configuration, no device touched */
    int tok = 0;
    if (mi_decoder_prefill(0, 0, &tok, 1, 0) != 0) return 4;    /* refused: no decoder, no device touched */
    printf("ok %d %d\n", (int)q[0], (int)p[0]);
    return 0;
}
''')
    exe = tmp_path / "abi"
    inc = os.path.join(ROOT, "include")
    libdir = os.path.dirname(mil.LIB_PATH)
    cmd = ["gcc", "-std=c11", "-Wall", "-Werror", "-pedantic", "-I", inc, str(src), "-o", str(exe),
           "-L", libdir, "-lmi_linear", f"-Wl,-rpath,{libdir}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.startswith("ok"), (r.returncode, r.stdout, r.stderr)


THREADS_PROGRAM = r'''
#include "mi_linear.h"
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
/* Host threads on the registry and the per-stream modes at once: each thread registers, looks up,
 * re-registers and unregisters its own keys and sets modes for its own stream handles, while all of
 * them also hammer a few shared keys.  The calls touch no device. */
enum { THREADS = 4, KEYS = 2000, ROUNDS = 20 };
static void* work(void* arg) {
    uintptr_t t = (uintptr_t)arg;
    long bad = 0;
    for (int r = 0; r < ROUNDS; ++r) {
        for (uintptr_t i = 1; i <= KEYS; ++i) {
            const void* mine = (const void*)((t + 1) * 0x1000000u + i * 64);
            const void* shared = (const void*)(0x900000u + (i % 7) * 64);
            bad += mi_register_int8_weight(mine, (const void*)0x10, 8, 64) != 1;
            bad += mi_weight_kind(mine) != 8;
            bad += mi_register_q4_weight(mine, (const void*)0x10, 8, 64) != 1;
            bad += mi_weight_kind(mine) != 4;
            mi_register_int8_weight(shared, (const void*)0x10, 4, 32);
            int k = mi_weight_kind(shared);
            bad += !(k == 8 || k == 0);
            mi_unregister_weight(shared);
            bad += mi_stream_set_modes((void*)mine, (int)(i & 1), 1) != 1;
            if (r + 1 < ROUNDS || (i & 3)) {
                bad += mi_unregister_weight(mine) != 1;
                bad += mi_weight_kind(mine) != 0;
                bad += mi_stream_set_modes((void*)mine, -1, -1) != 1;
            }
        }
    }
    return (void*)bad;
}
int main(void) {
    pthread_t th[THREADS];
    long bad = 0;
    for (uintptr_t t = 0; t < THREADS; ++t) pthread_create(&th[t], 0, work, (void*)t);
    for (int t = 0; t < THREADS; ++t) { void* r; pthread_join(th[t], &r); bad += (long)r; }
    long left = 0;
    for (uintptr_t t = 0; t < THREADS; ++t)
        for (uintptr_t i = 1; i <= KEYS; ++i) {
            const void* mine = (const void*)((t + 1) * 0x1000000u + i * 64);
            int k = mi_weight_kind(mine);
            if (i & 3) bad += k != 0; else { bad += k != 4; ++left; mi_unregister_weight(mine); }
        }
    printf("bad %ld left %ld\n", bad, left);
    return bad != 0;
}
'''


def test_host_threads_share_the_registry_and_the_stream_modes(tmp_path):
    """The reference's host is single threaded (QW/src/utils.cpp:63-66: plain statics); this library's
    registry and per-stream modes sit behind a mutex, which four threads exercise here without a GPU."""
    import subprocess
    src = tmp_path / "threads.c"
    src.write_text(THREADS_PROGRAM)
    exe = tmp_path / "threads"
    libdir = os.path.dirname(mil.LIB_PATH)
    cmd = ["gcc", "-std=c11", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
           "-L", libdir, "-lmi_linear", f"-Wl,-rpath,{libdir}", "-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip() == "bad 0 left 2000", (r.returncode, r.stdout, r.stderr[-2000:])
