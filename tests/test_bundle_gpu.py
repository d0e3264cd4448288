"""A bundle on disk -> device buffers -> registered weights -> pytorch_linear, on the GPU.

The load path of the reference: Weights::get_buffer (QW/src/weights.cpp:262-293) makes one device buffer
per tensor, the NNOPT_QUANT loop (LF/src/main.cpp:527-566) registers every 2-D int8 / q4_packed tensor that
has a scale sibling (Q4: K = scale columns * 32, :552-557), and from then on pytorch_linear on such a W takes
the quantised GEMV.  Here: mi_bundle_upload / mi_bundle_device_ptr / mi_bundle_close.  The bundles are the
ones the reference's own scripts wrote (tests/golden/bundle/), so reference-held bytes flow through the HIP
kernels; results are compared bit for bit with the oracle's GEMV on the mmap-ed host bytes."""
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

import oracle_lib as O
from helpers import ROOT, mil, synth_x

pytestmark = pytest.mark.gpu

G = os.path.join(ROOT, "tests", "golden", "bundle")
TAGS = ["int8", "q4", "int8_embed_alias", "q4_alias"]
KIND = {"int8": 8, "q4_packed": 4}


@pytest.fixture(scope="module")
def queue():
    assert mil.lib().mi_init(0) == 1, "no gfx950 device"
    mil.lib().mi_set_gemv_mode(0)          # reference evaluation order for every kind (bit-exact)
    q = mil.Queue()
    yield q
    q.finish()
    mil.lib().mi_set_gemv_mode(1)


def _quantised(meta, suffixes=(".scale",)):
    """name -> (scale name, N, K) for what the reference's loop registers."""
    t = meta["tensors"]
    out = {}
    for name, v in t.items():
        if v["dtype"] not in KIND or len(v["shape"]) != 2:
            continue
        sib = next((name + s for s in suffixes if name + s in t), None)
        if sib is None:
            continue
        if v["dtype"] == "int8":
            out[name] = (sib, v["shape"][0], v["shape"][1])
        elif len(t[sib]["shape"]) == 2:
            out[name] = (sib, v["shape"][0], t[sib]["shape"][1] * 32)
    return out


def _check_bundle(queue, bin_path, meta_path, suffixes=(".scale",)):
    meta = json.load(open(meta_path))
    want = _quantised(meta, suffixes)
    assert want, "the bundle holds quantised tensors"
    w = mil.Weights()
    assert w.load(bin_path, meta_path)
    assert w.upload() == len(want)
    assert w.upload() == len(want)          # a second call uploads and registers nothing twice
    ptrs = {}
    for name, v in meta["tensors"].items():
        dev = w.get_buffer(name)
        assert dev, name
        ptrs[name] = dev
        # every tensor is a device copy of its bytes in the file (get_buffer's CL_MEM_COPY_HOST_PTR)
        back = np.empty(v["size_bytes"], np.uint8)
        assert mil.lib().mi_memcpy_d2h(back.ctypes.data, dev, back.nbytes, None)
        host = w.get_host(name)
        assert np.array_equal(back, np.ascontiguousarray(host).view(np.uint8).reshape(-1)), name
        assert mil.lib().mi_weight_kind(dev) == (KIND[v["dtype"]] if name in want else 0), name
    assert len(set(ptrs.values())) == len(ptrs)
    for i, (name, (sib, N, K)) in enumerate(sorted(want.items())):
        print(f"bundle {os.path.basename(bin_path)} {name} N={N} K={K}", flush=True)
        x = synth_x(900 + i, K)
        xb, ob = mil.Buffer.from_host(x), mil.Buffer(N * 2)
        assert mil.pytorch_linear(queue, 1, N, K, xb, ptrs[name], ob)
        queue.finish()
        got = ob.read(np.uint16, (N,))
        Wh, sh = np.ascontiguousarray(w.get_host(name)), np.ascontiguousarray(w.get_host(sib)).view(np.uint16)
        if meta["tensors"][name]["dtype"] == "int8":
            ref = O.gemv_i8(x, Wh, sh)
        else:
            ref = O.gemv_q4(x, Wh, sh)
        assert np.array_equal(got, ref), f"{name}: {np.count_nonzero(got != ref)} of {N} differ"
        # N and K "must match the GEMV call site exactly" (LF/src/utils.h:126-128): the packed width is refused
        if meta["tensors"][name]["dtype"] == "q4_packed":
            assert not mil.pytorch_linear(queue, 1, N, K // 2, xb, ptrs[name], ob)
    # an fp16 tensor of the bundle goes through the same call as plain fp16 weights
    emb = "model.embed_tokens.weight"
    if meta["tensors"][emb]["dtype"] == "float16":
        N, K = meta["tensors"][emb]["shape"]
        x = synth_x(77, K)
        xb, ob = mil.Buffer.from_host(x), mil.Buffer(N * 2)
        assert mil.pytorch_linear(queue, 1, N, K, xb, ptrs[emb], ob)
        queue.finish()
        assert np.array_equal(ob.read(np.uint16, (N,)), O.gemv_f16(x, np.ascontiguousarray(w.get_host(emb))))
    w.close()
    for name in want:                       # the registry entries go with the bundle
        assert mil.lib().mi_weight_kind(ptrs[name]) == 0, name
    return len(want)


@pytest.mark.parametrize("tag", TAGS)
def test_reference_written_bundle_through_upload_registry_and_gemv(queue, tag):
    _check_bundle(queue, os.path.join(G, f"tiny.{tag}.bin"), os.path.join(G, f"tiny.{tag}.meta.json"))


def test_scales_spelling_of_lfm2_vl_bundles_registers_too(queue, tmp_path):
    """LV/scripts/quantize_int8.py:91-97 names the sibling "<name>.scales"."""
    meta = json.load(open(os.path.join(G, "tiny.int8.meta.json")))
    renamed = {}
    for name, v in meta["tensors"].items():
        renamed[name + "s" if name.endswith(".weight.scale") else name] = v
    meta["tensors"] = renamed
    mp = tmp_path / "vl.meta.json"
    mp.write_text(json.dumps(meta))
    bp = tmp_path / "vl.bin"
    shutil.copy(os.path.join(G, "tiny.int8.bin"), bp)
    assert _check_bundle(queue, str(bp), str(mp), suffixes=(".scales",)) == 9


def test_tensor_without_a_scale_sibling_stays_unregistered(queue, tmp_path):
    """`if (!weights.has_tensor(scale_name)) continue;` (LF/src/main.cpp:532, 547)."""
    meta = json.load(open(os.path.join(G, "tiny.q4.meta.json")))
    orphan = "model.layers.1.self_attn.k_proj.weight"
    meta["tensors"][orphan + ".lost"] = meta["tensors"].pop(orphan + ".scale")
    mp = tmp_path / "o.meta.json"
    mp.write_text(json.dumps(meta))
    w = mil.Weights()
    assert w.load(os.path.join(G, "tiny.q4.bin"), str(mp))
    assert w.upload() == 8
    assert mil.lib().mi_weight_kind(w.get_buffer(orphan)) == 0
    assert mil.lib().mi_weight_kind(w.get_buffer("model.layers.1.self_attn.q_proj.weight")) == 4
    w.close()


C_PROGRAM = r"""
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "mi_linear.h"
/* A C caller of the load path: open, upload, look a weight up by name, one GEMV, close. */
int main(int argc, char** argv) {
    if (argc != 3) return 2;
    if (!mi_init(0)) return 3;
    void* b = mi_bundle_open(argv[1], argv[2]);
    if (!b) return 4;
    int registered = mi_bundle_upload(b);
    const char* name = "model.layers.0.feed_forward.w2.weight";
    const void* host; size_t bytes; const char* dtype; int ndim; int64_t shape[4];
    if (!mi_bundle_tensor(b, name, &host, &bytes, &dtype, &ndim, shape)) return 5;
    void* W = mi_bundle_device_ptr(b, name);
    int N = (int)shape[0], K = strcmp(dtype, "q4_packed") == 0 ? (int)shape[1] * 2 : (int)shape[1];
    uint16_t* x = calloc((size_t)K, 2);
    x[5] = 0x3C00;                                   /* e_5: the product is column 5 of the dequantised W */
    void* xd = mi_malloc((size_t)K * 2);
    void* yd = mi_malloc((size_t)N * 2);
    uint16_t* y = malloc((size_t)N * 2);
    if (!mi_memcpy_h2d(xd, x, (size_t)K * 2, NULL)) return 6;
    if (!mi_linear(NULL, 1, N, K, xd, W, yd)) return 7;
    if (!mi_memcpy_d2h(y, yd, (size_t)N * 2, NULL)) return 8;
    printf("%d %d %d %d", registered, mi_weight_kind(W), N, K);
    for (int n = 0; n < N; ++n) printf(" %u", (unsigned)y[n]);
    printf("\n");
    mi_bundle_close(b);
    printf("%d\n", mi_weight_kind(W));
    return 0;
}
"""


@pytest.mark.parametrize("tag", ["int8", "q4"])
def test_c_caller_of_the_load_path(tmp_path, tag):
    src = tmp_path / "load.c"
    src.write_text(C_PROGRAM)
    exe = tmp_path / "load"
    libdir = os.path.dirname(mil.LIB_PATH)
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src),
                           "-o", str(exe), "-L", libdir, "-lmi_linear", f"-Wl,-rpath,{libdir}"])
    out = subprocess.run([str(exe), os.path.join(G, f"tiny.{tag}.bin"), os.path.join(G, f"tiny.{tag}.meta.json")],
                         check=True, capture_output=True, text=True, timeout=120).stdout.split("\n")
    head = [int(v) for v in out[0].split()]
    meta = json.load(open(os.path.join(G, f"tiny.{tag}.meta.json")))
    assert head[:4] == [len(_quantised(meta)), 8 if tag == "int8" else 4, 64, 96]
    assert int(out[1]) == 0
    w = mil.Weights()
    assert w.load(os.path.join(G, f"tiny.{tag}.bin"), os.path.join(G, f"tiny.{tag}.meta.json"))
    name = "model.layers.0.feed_forward.w2.weight"
    Wh, sh = w.get_host(name), w.get_host(name + ".scale")
    if tag == "int8":
        col = (Wh[:, 5].astype(np.float32) * sh.astype(np.float32)).astype(np.float16)
    else:
        nib = (Wh[:, 2] >> 4).astype(np.float32) - 8          # element 5 = high nibble of byte 2
        col = (nib * sh[:, 0].astype(np.float32)).astype(np.float16)
    assert np.array_equal(np.array(head[4:], np.uint16), col.view(np.uint16))
    w.close()
