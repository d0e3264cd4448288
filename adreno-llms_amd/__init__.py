"""Host-side mirror of the reference's linear-op interface over libmi_linear.so.

The names and argument meaning follow the reference's C++ host layer
(src/models/qwen2-5-0-5b/src/utils.h:119-159, src/models/lfm2-5-350m/src/utils.h:122-145,
src/models/qwen2-5-0-5b/src/weights.h) so that tests read like calls into the
reference: `pytorch_linear(queue, M, N, K, x, W, out)` returns True when work was
enqueued, `nnopt_register_int8_weight(W, scale, N, K)` files a weight under its
handle, `Weights.load / get_buffer / get_dtype / get_shape / all_keys` read a
`.bin` + `.meta.json` bundle.  A `Buffer` stands where the reference holds a
`cl_mem`, a `Queue` where it holds a `cl_command_queue`.

Everything computes on the GPU through the C ABI declared in include/mi_linear.h.
There is no CPU fallback: loading fails loudly when the HIP library is missing.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi_linear.so")

_vp, _i, _sz = C.c_void_p, C.c_int, C.c_size_t

_SIGNATURES = {
    "mi_init": (_i, [_i]),
    "mi_device_arch": (C.c_char_p, []),
    "mi_device_cus": (_i, []),
    "mi_malloc": (_vp, [_sz]),
    "mi_free": (_i, [_vp]),
    "mi_memcpy_h2d": (_i, [_vp, _vp, _sz, _vp]),
    "mi_memcpy_d2h": (_i, [_vp, _vp, _sz, _vp]),
    "mi_memcpy_d2d": (_i, [_vp, _vp, _sz, _vp]),
    "mi_memset": (_i, [_vp, _i, _sz, _vp]),
    "mi_stream_create": (_vp, []),
    "mi_stream_destroy": (_i, [_vp]),
    "mi_stream_sync": (_i, [_vp]),
    "mi_event_create": (_vp, []),
    "mi_event_destroy": (_i, [_vp]),
    "mi_event_record": (_i, [_vp, _vp]),
    "mi_event_sync": (_i, [_vp]),
    "mi_event_elapsed_ms": (C.c_float, [_vp, _vp]),
    "mi_register_int8_weight": (_i, [_vp, _vp, _i, _i]),
    "mi_register_q4_weight": (_i, [_vp, _vp, _i, _i]),
    "mi_unregister_weight": (_i, [_vp]),
    "mi_weight_kind": (_i, [_vp]),
    "mi_linear": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
    "mi_linear_batch": (_i, [_vp, _vp, _i]),
    "mi_graph_begin": (_i, [_vp]),
    "mi_graph_end": (_vp, [_vp]),
    "mi_graph_launch": (_i, [_vp, _vp]),
    "mi_graph_destroy": (_i, [_vp]),
    "mi_linear_add": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
    "mi_linear_gate_up_silu": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp]),
    "mi_linear_silu_gate": (_i, [_vp, _i, _i, _vp, _vp, _vp]),
    "mi_dequant_int8_to_fp16": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "mi_unpack_q4_to_int8": (_i, [_vp, _vp, _i, _i, _vp]),
    "mi_decoder_create": (_vp, [_vp, _vp]),
    "mi_decoder_destroy": (_i, [_vp]),
    "mi_decoder_reset": (_i, [_vp, _vp, _i, _i]),
    "mi_decoder_set_token": (_i, [_vp, _vp, _i]),
    "mi_decoder_step": (_i, [_vp, _vp]),
    "mi_decoder_set_attention_splits": (_i, [_vp, _i]),
    "mi_decoder_prefill": (_i, [_vp, _vp, C.POINTER(_i), _i, _i]),
    "mi_decoder_reserve_prompt": (_i, [_vp, _vp, _i]),
    "mi_decoder_read": (_i, [_vp, _vp, C.POINTER(_i), C.POINTER(_i)]),
    "mi_decoder_logits": (_vp, [_vp]),
    "mi_decoder_buffer": (_vp, [_vp, _i]),
    "mi_argmax_f16": (_i, [_vp, _vp, _i, _i, _vp]),
    "mi_linear_argmax": (_i, [_vp, _i, _i, _vp, _vp, _vp, _i, _vp]),
    "mi_linear_argmax_static": (_i, [_vp, _i, _i, _vp, _vp, _vp, _i, _vp]),
    "mi_stream_set_modes": (_i, [_vp, _i, _i]),
    "mi_stream_read_probe": (_i, [_vp, _vp, C.c_size_t, _vp]),
    "mi_linear_plan": (_i, [_vp, _i, _i, _i, _vp, _vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "mi_set_gemm_mode": (None, [_i]),
    "mi_set_gemv_mode": (None, [_i]),
    "mi_quantize_int8": (_i, [_vp, _i, _i, _vp, _vp]),
    "mi_quantize_q4": (_i, [_vp, _i, _i, _vp, _vp]),
    "mi_f16_to_f32": (C.c_float, [C.c_uint16]),
    "mi_f32_to_f16": (C.c_uint16, [C.c_float]),
    "mi_synth_normal_f16": (None, [C.c_uint64, C.c_double, _sz, _vp]),
    "mi_bundle_open": (_vp, [C.c_char_p, C.c_char_p]),
    "mi_bundle_close": (None, [_vp]),
    "mi_bundle_count": (_i, [_vp]),
    "mi_bundle_name": (C.c_char_p, [_vp, _i]),
    "mi_bundle_tensor": (_i, [_vp, C.c_char_p, C.POINTER(_vp), C.POINTER(_sz), C.POINTER(C.c_char_p),
                              C.POINTER(_i), C.POINTER(C.c_int64)]),
    "mi_bundle_upload": (_i, [_vp]),
    "mi_bundle_device_ptr": (_vp, [_vp, C.c_char_p]),
}


def load_library(path=LIB_PATH):
    """dlopen the HIP library and type its entry points.  Raises if it is not built."""
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: build it with `python adreno-llms_amd/build.py` "
            "(there is no CPU fallback for this path)")
    lib = C.CDLL(path)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = load_library()
    return _lib


def _ptr(a):
    return a.ctypes.data_as(_vp)


# ----------------------------------------------------------------------------- runtime

class Queue:
    """An in-order HIP stream (the reference's cl_command_queue)."""

    def __init__(self, default=False):
        self.handle = None if default else lib().mi_stream_create()
        if not default and not self.handle:
            raise RuntimeError("mi_stream_create failed")

    def finish(self):                                   # clFinish
        if not lib().mi_stream_sync(self.handle):
            raise RuntimeError("mi_stream_sync failed")

    def __del__(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.mi_stream_destroy(self.handle)
            self.handle = None


class Buffer:
    """A device allocation (the reference's cl_mem)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = lib().mi_malloc(self.nbytes)
        if not self.ptr:
            raise MemoryError(f"mi_malloc({nbytes}) failed")

    @classmethod
    def from_host(cls, array):
        a = np.ascontiguousarray(array)
        b = cls(a.nbytes)
        b.write(a)
        return b

    def write(self, array, queue=None):
        a = np.ascontiguousarray(array)
        assert a.nbytes <= self.nbytes
        if not lib().mi_memcpy_h2d(self.ptr, _ptr(a), a.nbytes, queue.handle if queue else None):
            raise RuntimeError("mi_memcpy_h2d failed")

    def read(self, dtype, shape, queue=None):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        if not lib().mi_memcpy_d2h(_ptr(out), self.ptr, out.nbytes, queue.handle if queue else None):
            raise RuntimeError("mi_memcpy_d2h failed")
        return out

    def release(self):                                   # clReleaseMemObject
        if self.ptr and _lib is not None:
            _lib.mi_free(self.ptr)
        self.ptr = None

    def __del__(self):
        self.release()


def _h(buf):
    return buf.ptr if isinstance(buf, Buffer) else buf


def _q(queue):
    return queue.handle if isinstance(queue, Queue) else queue


class Event:
    def __init__(self):
        self.handle = lib().mi_event_create()

    def record(self, queue=None):
        lib().mi_event_record(self.handle, _q(queue))

    def synchronize(self):
        lib().mi_event_sync(self.handle)

    def elapsed_ms(self, stop):
        return float(lib().mi_event_elapsed_ms(self.handle, stop.handle))

    def __del__(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.mi_event_destroy(self.handle)
            self.handle = None


# ------------------------------------------------------------------ the linear-op API

def pytorch_linear(queue, M, N, K, x, W, out):
    """out[M,N] = x[M,K] @ W[N,K]^T (QW/src/utils.h:119-121).  True = enqueued."""
    return bool(lib().mi_linear(_q(queue), M, N, K, _h(x), _h(W), _h(out)))


class LinearCall(C.Structure):
    _fields_ = [("M", _i), ("N", _i), ("K", _i), ("x", _vp), ("W", _vp), ("out", _vp)]


def make_calls(calls):
    """[(M, N, K, x, W, out), ...] -> ctypes array for linear_batch."""
    arr = (LinearCall * len(calls))()
    for i, (M, N, K, x, W, out) in enumerate(calls):
        arr[i] = LinearCall(M, N, K, _h(x), _h(W), _h(out))
    return arr


def linear_batch(queue, call_array):
    """Enqueue a prepared list of pytorch_linear calls in order; returns how many were enqueued."""
    return lib().mi_linear_batch(_q(queue), call_array, len(call_array))


class Graph:
    """Record / replay of the launches enqueued on a queue (a HIP graph)."""

    def __init__(self, queue):
        self.queue = queue
        self.handle = None

    def __enter__(self):
        if not lib().mi_graph_begin(_q(self.queue)):
            raise RuntimeError("mi_graph_begin failed")
        return self

    def __exit__(self, *exc):
        self.handle = lib().mi_graph_end(_q(self.queue))
        if not self.handle and exc[0] is None:
            raise RuntimeError("mi_graph_end failed")

    def launch(self, queue=None):
        if not lib().mi_graph_launch(self.handle, _q(queue or self.queue)):
            raise RuntimeError("mi_graph_launch failed")

    def __del__(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.mi_graph_destroy(self.handle)
            self.handle = None


def pytorch_linear_add(queue, M, N, K, x, W, residual_inout):
    """residual += W x, M == 1 only (QW/src/utils.h:133-135).  False = not taken."""
    return bool(lib().mi_linear_add(_q(queue), M, N, K, _h(x), _h(W), _h(residual_inout)))


def fused_gate_up_silu_m1(queue, N, K, x, Wg, Wu, out):
    """out = silu(Wg x) * (Wu x) (QW/src/utils.h:157-159).  False = not taken."""
    return bool(lib().mi_linear_gate_up_silu(_q(queue), N, K, _h(x), _h(Wg), _h(Wu), _h(out)))


def pytorch_linear_silu_gate_fused(queue, N, K, x, W3, gate_inout):
    """gate_inout = silu(gate_inout) * (W3 x) (LF/src/utils.h:140-142).  False = not taken."""
    return bool(lib().mi_linear_silu_gate(_q(queue), N, K, _h(x), _h(W3), _h(gate_inout)))


def nnopt_register_int8_weight(W_int8, scale_fp16, N, K):
    """LF/src/utils.h:129."""
    return bool(lib().mi_register_int8_weight(_h(W_int8), _h(scale_fp16), N, K))


def nnopt_register_q4_weight(W_q4, scale_fp16, N, K):
    """LF/src/utils.h:134; K is the unpacked K."""
    return bool(lib().mi_register_q4_weight(_h(W_q4), _h(scale_fp16), N, K))


def nnopt_unregister_weight(W):
    return bool(lib().mi_unregister_weight(_h(W)))


def dequant_int8_weight_to_fp16(queue, W_int8, scale_fp16, N, K, out_fp16):
    """LV/src/utils.cpp:594-634."""
    return bool(lib().mi_dequant_int8_to_fp16(_q(queue), _h(W_int8), _h(scale_fp16), N, K, _h(out_fp16)))


def unpack_q4_to_int8(queue, W_q4, N, K, out_int8):
    return bool(lib().mi_unpack_q4_to_int8(_q(queue), _h(W_q4), N, K, _h(out_int8)))


def argmax_f16(queue, logits, N, token_out, num_partials=32):
    """argmax_partial + argmax_finalize (QW/kernels/gemv_m1.cl:198-280); token_out: int32 on the device."""
    return bool(lib().mi_argmax_f16(_q(queue), _h(logits), N, num_partials, _h(token_out)))


def pytorch_linear_argmax(queue, N, K, x, W, logits, token_out, num_partials=32):
    """The lm_head of a greedy step: dispatch_lm_head_argmax (QW/src/model.cpp:436-482)."""
    return bool(lib().mi_linear_argmax(_q(queue), N, K, _h(x), _h(W), _h(logits), num_partials, _h(token_out)))


def linear_plan(queue, M, N, K, x, W):
    """(kernel, rows of x per block, slices of K) mi_linear would use; kernel 0 = GEMV rows, 1 = wide MFMA kernel,
    2 / 3 = tile kernels, 4 = the streaming kernel for up to 64 rows of x, 5 = the kernel with 256 x 256 blocks."""
    tr, ks = C.c_int(0), C.c_int(1)
    kern = lib().mi_linear_plan(_q(queue), M, N, K, _h(x), _h(W), C.byref(tr), C.byref(ks))
    return kern, tr.value, ks.value


def pytorch_linear_argmax_static(queue, N, K, x, W, logits, token_out, num_partials=32):
    """pytorch_linear_argmax for callers that cannot allocate: the kernels' scratch is an array
    inside the library (mi_linear_argmax_static); works on any stream."""
    return bool(lib().mi_linear_argmax_static(_q(queue), N, K, _h(x), _h(W), _h(logits), num_partials,
                                              _h(token_out)))


class DecoderConfig(C.Structure):
    """mi_decoder_config (include/mi_decode.h)."""
    _fields_ = [(n, _i) for n in ("hidden", "inter", "n_heads", "n_kv_heads", "head_dim", "n_layers", "vocab",
                                  "max_pos")] + [("rms_eps", C.c_float), ("rope_theta", C.c_float)]


class DecoderWeights(C.Structure):
    """mi_decoder_weights (include/mi_decode.h)."""
    _fields_ = [("embed", _vp), ("final_norm", _vp), ("lm_head", _vp)] + \
               [(n, C.POINTER(_vp)) for n in ("in_norm", "post_norm", "bq", "bk", "bv", "wq", "wk", "wv", "wo",
                                              "wgate", "wup", "wdown")]


class Decoder:
    """Greedy decoding on the device (Model::forward_greedy and the decode loop, QW/src/model.cpp:387-500).

    cfg: dict with the DecoderConfig fields; weights: dict name -> Buffer (embed, final_norm, lm_head)
    or list of Buffers per layer (the other DecoderWeights fields)."""

    def __init__(self, cfg, weights):
        c = DecoderConfig()
        for name, _ in DecoderConfig._fields_:
            setattr(c, name, cfg[name])
        w = DecoderWeights()
        self._keep = [weights]
        for name in ("embed", "final_norm", "lm_head"):
            setattr(w, name, _h(weights[name]))
        for name, _ in DecoderWeights._fields_[3:]:
            arr = (_vp * cfg["n_layers"])(*[_h(b) for b in weights[name]])
            self._keep.append(arr)
            setattr(w, name, arr)
        self.handle = lib().mi_decoder_create(C.byref(c), C.byref(w))
        if not self.handle:
            raise RuntimeError("mi_decoder_create failed")

    def reset(self, queue, pos, token):
        return bool(lib().mi_decoder_reset(self.handle, _q(queue), pos, token))

    def set_token(self, queue, token):
        return bool(lib().mi_decoder_set_token(self.handle, _q(queue), token))

    def step(self, queue):
        return bool(lib().mi_decoder_step(self.handle, _q(queue)))

    def set_attention_splits(self, splits):
        """0 / 1: the reference-order attention (default); 2..32: a head's keys split over that many blocks."""
        return bool(lib().mi_decoder_set_attention_splits(self.handle, int(splits)))

    def prefill(self, queue, tokens, pos0=0):
        """A prompt at once (Model::forward with seq_len = len(tokens), QW/src/model.cpp:243-376)."""
        arr = (_i * len(tokens))(*[int(t) for t in tokens])
        return bool(lib().mi_decoder_prefill(self.handle, _q(queue), arr, len(tokens), pos0))

    def reserve_prompt(self, queue, max_tokens):
        """Room (and the stacked projection matrices) for prompts of up to max_tokens tokens, made now."""
        return bool(lib().mi_decoder_reserve_prompt(self.handle, _q(queue), int(max_tokens)))

    def read(self, queue):
        pos, tok = _i(), _i()
        if not lib().mi_decoder_read(self.handle, _q(queue), C.byref(pos), C.byref(tok)):
            raise RuntimeError("mi_decoder_read failed")
        return pos.value, tok.value

    @property
    def logits_ptr(self):
        return lib().mi_decoder_logits(self.handle)

    def close(self):
        if self.handle and _lib is not None:
            _lib.mi_decoder_destroy(self.handle)
        self.handle = None

    def __del__(self):
        self.close()


# ------------------------------------------------------------------- offline tools

def quantize_int8(w_fp16):
    """Rows of fp16 -> (int8 [N,K], fp16 scale [N]); LF/scripts/quantize_weights.py:53-57."""
    w = np.ascontiguousarray(w_fp16, dtype=np.float16)
    N, K = w.shape
    q = np.empty((N, K), np.int8)
    s = np.empty(N, np.float16)
    if not lib().mi_quantize_int8(_ptr(w), N, K, _ptr(q), _ptr(s)):
        raise ValueError("mi_quantize_int8 failed")
    return q, s


def quantize_q4(w_fp16):
    """Rows of fp16 -> (u8 [N,K/2], fp16 scale [N,K/32]); LF/scripts/quantize_q4.py:62-82."""
    w = np.ascontiguousarray(w_fp16, dtype=np.float16)
    N, K = w.shape
    if K % 32:
        raise RuntimeError(f"Q4 requires K divisible by 32, got {K}")
    p = np.empty((N, K // 2), np.uint8)
    s = np.empty((N, K // 32), np.float16)
    if not lib().mi_quantize_q4(_ptr(w), N, K, _ptr(p), _ptr(s)):
        raise ValueError("mi_quantize_q4 failed")
    return p, s


def synth_normal_f16(seed, sigma, shape):
    """Seeded N(0, sigma) tensor rounded to fp16 (counter-based, thread-count independent)."""
    out = np.empty(shape, np.float16)
    lib().mi_synth_normal_f16(int(seed), float(sigma), out.size, _ptr(out))
    return out


# ----------------------------------------------------------------------- bundles

class Weights:
    """.bin + .meta.json bundle (QW/src/weights.h; QW/src/weights.cpp:165-293)."""

    def __init__(self):
        self._h = None

    def load(self, bin_path, meta_path):
        self._h = lib().mi_bundle_open(os.fsencode(bin_path), os.fsencode(meta_path))
        return bool(self._h)

    def all_keys(self):
        return [lib().mi_bundle_name(self._h, i).decode() for i in range(lib().mi_bundle_count(self._h))]

    def _tensor(self, key):
        host, size, dtype, ndim = _vp(), _sz(), C.c_char_p(), _i()
        shape = (C.c_int64 * 4)()
        ok = lib().mi_bundle_tensor(self._h, key.encode(), C.byref(host), C.byref(size), C.byref(dtype),
                                    C.byref(ndim), shape)
        if not ok:
            return None
        return host.value, size.value, dtype.value.decode(), [int(shape[i]) for i in range(ndim.value)]

    def has_tensor(self, key):
        return self._tensor(key) is not None

    def get_dtype(self, key):
        t = self._tensor(key)
        return t[2] if t else ""

    def get_shape(self, key):
        t = self._tensor(key)
        return t[3] if t else []

    def get_size_bytes(self, key):
        t = self._tensor(key)
        return t[1] if t else 0

    def get_host(self, key):
        """Host view of the mmap-ed tensor bytes as a numpy array of its dtype."""
        t = self._tensor(key)
        if not t:
            return None
        host, size, dtype, shape = t
        np_dtype = {"float16": np.float16, "int8": np.int8, "q4_packed": np.uint8}.get(dtype, np.float32)
        raw = (C.c_uint8 * size).from_address(host)
        return np.frombuffer(raw, dtype=np_dtype).reshape(shape)

    def upload(self):
        """Copies every tensor to the GPU and registers the quantised ones
        (LF/src/main.cpp:527-566).  Returns the number of registered weights."""
        return lib().mi_bundle_upload(self._h)

    def get_buffer(self, key):
        return lib().mi_bundle_device_ptr(self._h, key.encode())

    def close(self):
        if self._h and _lib is not None:
            _lib.mi_bundle_close(self._h)
        self._h = None

    def __del__(self):
        self.close()
