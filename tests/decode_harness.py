"""Test harness for the greedy-decode token check: builds a seeded random-init
Qwen2-shaped model (int8 per-row projections, fp16 embedding tied to an int8 lm_head) and
drives oracle/decode.c, whose projections go through a callback."""
import ctypes as C

import numpy as np

import oracle_lib as O
from helpers import mil

QWEN25_05B = dict(hidden=896, inter=4864, n_heads=14, n_kv_heads=2, head_dim=64, n_layers=24,
                  vocab=151936, max_pos=64, rms_eps=1e-6, rope_theta=1000000.0)
TINY = dict(hidden=64, inter=128, n_heads=4, n_kv_heads=2, head_dim=16, n_layers=2,
            vocab=512, max_pos=48, rms_eps=1e-6, rope_theta=10000.0)
# SmolLM2-135M widths, cut to 3 layers and a small vocabulary: K = 576 and 1536
SMOL = dict(hidden=576, inter=1536, n_heads=9, n_kv_heads=3, head_dim=64, n_layers=3,
            vocab=4096, max_pos=48, rms_eps=1e-5, rope_theta=100000.0)
PROMPT = [785, 11079, 6439, 518, 279, 220]       # QW/reference/test_input_ids.bin

_PP16 = C.POINTER(C.POINTER(C.c_uint16))


class OrcModel(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("hidden", "inter", "n_heads", "n_kv_heads", "head_dim", "n_layers",
                                        "vocab", "max_pos")] + \
               [("rms_eps", C.c_float), ("rope_theta", C.c_float),
                ("embed", C.c_void_p), ("final_norm", C.c_void_p),
                ("in_norm", C.POINTER(C.c_void_p)), ("post_norm", C.POINTER(C.c_void_p)),
                ("bq", C.POINTER(C.c_void_p)), ("bk", C.POINTER(C.c_void_p)), ("bv", C.POINTER(C.c_void_p)),
                ("w8", C.POINTER(C.c_void_p)), ("wscale", C.POINTER(C.c_void_p))]


LINEAR_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p)

_lib = O.lib
_lib.orc_decoder_new.restype = C.c_void_p
_lib.orc_decoder_new.argtypes = [C.POINTER(OrcModel), C.c_int]
_lib.orc_decoder_free.argtypes = [C.c_void_p]
_lib.orc_decoder_logits.restype = C.c_void_p
_lib.orc_decoder_logits.argtypes = [C.c_void_p]
_lib.orc_decoder_step.restype = C.c_int
_lib.orc_decoder_step.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]


class Model:
    """Seeded random-init weights: W ~ N(0, 0.02) fp16 then int8 per row; norms 1 + N(0, 0.02);
    q/k/v biases N(0, 0.02); embedding fp16 N(0, 0.02); lm_head int8, independent of the embedding."""

    def __init__(self, cfg, seed=2024):
        self.cfg = dict(cfg)
        c = self.cfg
        qd, kvd = c["n_heads"] * c["head_dim"], c["n_kv_heads"] * c["head_dim"]
        self.shapes = []
        for _ in range(c["n_layers"]):
            self.shapes += [(qd, c["hidden"]), (kvd, c["hidden"]), (kvd, c["hidden"]), (c["hidden"], qd),
                            (c["inter"], c["hidden"]), (c["inter"], c["hidden"]), (c["hidden"], c["inter"])]
        self.shapes.append((c["vocab"], c["hidden"]))
        s = seed * 1000
        self.embed = mil.synth_normal_f16(s, 0.02, (c["vocab"], c["hidden"]))
        self.w8, self.ws = [], []
        for i, (N, K) in enumerate(self.shapes[:-1]):
            q, sc = mil.quantize_int8(mil.synth_normal_f16(s + 1 + i, 0.02, (N, K)))
            self.w8.append(q)
            self.ws.append(sc)
        # The lm_head is NOT tied to the embedding here: with random-init weights a tied head
        # makes "repeat the last token" a fixed point with a wide margin (the residual stream
        # is dominated by the token's own embedding), and a constant token list would check
        # nothing.  An independent head turns the model into a pseudo-random map over the
        # vocabulary with small top-1/top-2 margins, which is what stresses the GEMV order.
        q, sc = mil.quantize_int8(mil.synth_normal_f16(s + 400, 0.02, (c["vocab"], c["hidden"])))
        self.w8.append(q)
        self.ws.append(sc)
        one = np.float16(1.0)
        L = c["n_layers"]
        self.in_norm = [one + mil.synth_normal_f16(s + 500 + l, 0.02, (c["hidden"],)) for l in range(L)]
        self.post_norm = [one + mil.synth_normal_f16(s + 600 + l, 0.02, (c["hidden"],)) for l in range(L)]
        self.final_norm = one + mil.synth_normal_f16(s + 700, 0.02, (c["hidden"],))
        self.bq = [mil.synth_normal_f16(s + 800 + l, 0.02, (qd,)) for l in range(L)]
        self.bk = [mil.synth_normal_f16(s + 900 + l, 0.02, (kvd,)) for l in range(L)]
        self.bv = [mil.synth_normal_f16(s + 950 + l, 0.02, (kvd,)) for l in range(L)]

    def _ptrs(self, arrays):
        arr = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
        return arr

    def c_struct(self):
        c = self.cfg
        m = OrcModel()
        for k in ("hidden", "inter", "n_heads", "n_kv_heads", "head_dim", "n_layers", "vocab", "max_pos"):
            setattr(m, k, c[k])
        m.rms_eps, m.rope_theta = c["rms_eps"], c["rope_theta"]
        m.embed, m.final_norm = self.embed.ctypes.data, self.final_norm.ctypes.data
        self._keep = [self._ptrs(x) for x in (self.in_norm, self.post_norm, self.bq, self.bk, self.bv,
                                              self.w8, self.ws)]
        (m.in_norm, m.post_norm, m.bq, m.bk, m.bv, m.w8, m.wscale) = self._keep
        return m


def greedy(model, prompt, n_new, linear_cb=None, threads=O.THREADS, last_logits=None):
    """Feeds the prompt token by token, then decodes n_new tokens greedily.
    Returns (tokens, margins); linear_cb(index, x_ptr, y_ptr) replaces the oracle GEMV.
    last_logits: a uint16 array of vocab entries that receives the logits of the last step
    that produced a listed token."""
    cs = model.c_struct()
    dec = _lib.orc_decoder_new(C.byref(cs), threads)
    fn = LINEAR_FN(lambda ctx, idx, x, y: linear_cb(idx, x, y)) if linear_cb else None
    fn_ptr = C.cast(fn, C.c_void_p) if fn else None
    margin = C.c_float()
    toks, margins, pos, nxt = [], [], 0, -1
    try:
        for t in prompt:
            nxt = _lib.orc_decoder_step(dec, int(t) % model.cfg["vocab"], pos, fn_ptr, None, C.byref(margin))
            pos += 1
        for i in range(n_new):
            toks.append(nxt)
            margins.append(margin.value)
            if i == n_new - 1:
                if last_logits is not None:
                    src = (C.c_uint16 * model.cfg["vocab"]).from_address(_lib.orc_decoder_logits(dec))
                    last_logits[:] = np.ctypeslib.as_array(src)
                break
            nxt = _lib.orc_decoder_step(dec, nxt, pos, fn_ptr, None, C.byref(margin))
            pos += 1
    finally:
        _lib.orc_decoder_free(dec)
    return toks, margins


class KindModel(Model):
    """The same model with every projection stored as fp16 ("f16") or block-32 Q4 ("q4") instead of
    int8: the CPU harness reaches the matching oracle GEMV through the callback, the device decoder
    gets the weights registered (or not, for fp16) accordingly."""

    def __init__(self, cfg, kind, seed=2024):
        super().__init__(cfg, seed)
        assert kind in ("f16", "q4")
        self.kind = kind
        s = seed * 1000
        self.wf, self.wq4 = [], []
        for i, (N, K) in enumerate(self.shapes):
            w = mil.synth_normal_f16(s + 1 + (i if i < len(self.shapes) - 1 else 399), 0.02, (N, K))
            if kind == "f16":
                self.wf.append(w)
            else:
                self.wq4.append(mil.quantize_q4(w))

    def oracle_cb(self):
        def cb(idx, x_ptr, y_ptr):
            N, K = self.shapes[idx]
            x = np.ctypeslib.as_array((C.c_uint16 * K).from_address(x_ptr))
            y = np.ctypeslib.as_array((C.c_uint16 * N).from_address(y_ptr))
            if self.kind == "f16":
                y[:] = O.gemv_f16(x.view(np.float16), self.wf[idx])
            else:
                p, sc = self.wq4[idx]
                y[:] = O.gemv_q4(x.view(np.float16), p, sc.view(np.uint16))
        return cb


class GpuLinear:
    """The library behind the callback: weights resident and registered once, x up, y down."""

    def __init__(self, model, queue):
        self.model, self.queue = model, queue
        self.W = [mil.Buffer.from_host(q) for q in model.w8]
        self.S = [mil.Buffer.from_host(s) for s in model.ws]
        for (N, K), w, s in zip(model.shapes, self.W, self.S):
            assert mil.nnopt_register_int8_weight(w, s, N, K)
        kmax = max(K for _, K in model.shapes)
        nmax = max(N for N, _ in model.shapes)
        self.x, self.y = mil.Buffer(kmax * 2), mil.Buffer(nmax * 2)
        self.calls = 0

    def __call__(self, idx, x_ptr, y_ptr):
        N, K = self.model.shapes[idx]
        L = mil.lib()
        assert L.mi_memcpy_h2d(self.x.ptr, x_ptr, K * 2, self.queue.handle)
        assert mil.pytorch_linear(self.queue, 1, N, K, self.x, self.W[idx], self.y)
        assert L.mi_memcpy_d2h(y_ptr, self.y.ptr, N * 2, self.queue.handle)
        self.calls += 1

    def close(self):
        for w in self.W:
            mil.nnopt_unregister_weight(w)


class GpuDecoder:
    """The whole step on the device (mi_decoder_*): weights uploaded once, tokens read back only
    to build the list that is compared."""

    def __init__(self, model, queue):
        c = model.cfg
        self.model, self.queue = model, queue
        kind = getattr(model, "kind", "i8")
        if kind == "f16":
            self.W, self.S = [mil.Buffer.from_host(w) for w in model.wf], []
        elif kind == "q4":
            self.W = [mil.Buffer.from_host(p) for p, _ in model.wq4]
            self.S = [mil.Buffer.from_host(sc) for _, sc in model.wq4]
            for (N, K), w, s in zip(model.shapes, self.W, self.S):
                assert mil.nnopt_register_q4_weight(w, s, N, K)
        else:
            self.W = [mil.Buffer.from_host(q) for q in model.w8]
            self.S = [mil.Buffer.from_host(s) for s in model.ws]
            for (N, K), w, s in zip(model.shapes, self.W, self.S):
                assert mil.nnopt_register_int8_weight(w, s, N, K)
        up = lambda arrs: [mil.Buffer.from_host(a) for a in arrs]
        L = c["n_layers"]
        self.bufs = dict(embed=mil.Buffer.from_host(model.embed), final_norm=mil.Buffer.from_host(model.final_norm),
                         lm_head=self.W[-1], in_norm=up(model.in_norm), post_norm=up(model.post_norm),
                         bq=up(model.bq), bk=up(model.bk), bv=up(model.bv))
        for j, name in enumerate(("wq", "wk", "wv", "wo", "wgate", "wup", "wdown")):
            self.bufs[name] = [self.W[l * 7 + j] for l in range(L)]
        self.dec = mil.Decoder(c, self.bufs)

    def greedy(self, prompt, n_new, graph=False):
        q, d = self.queue, self.dec
        vocab = self.model.cfg["vocab"]
        assert d.reset(q, 0, int(prompt[0]) % vocab)
        g = None
        if graph:
            d.step(q)                                # warm-up outside the capture (first-use setup of the kernels)
            q.finish()
            assert d.reset(q, 0, int(prompt[0]) % vocab)
            with mil.Graph(q) as g:
                assert d.step(q)
        run = (lambda: g.launch()) if graph else (lambda: d.step(q))
        for t in prompt[1:]:
            run()
            assert d.set_token(q, int(t) % vocab)    # prompt feeding: the model's own prediction is overridden
        toks = []
        for _ in range(n_new):
            run()
            toks.append(d.read(q)[1])
        return toks

    def logits(self):
        """Logits of the last step, as stored by the lm_head (uint16 bit patterns)."""
        vocab = self.model.cfg["vocab"]
        out = np.empty(vocab, np.uint16)
        self.queue.finish()
        assert mil.lib().mi_memcpy_d2h(out.ctypes.data, self.dec.logits_ptr, vocab * 2, self.queue.handle)
        self.queue.finish()
        return out

    def close(self):
        self.dec.close()
        for w in self.W:
            mil.nnopt_unregister_weight(w)
