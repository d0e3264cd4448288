"""Pins oracle/decode.c (the decode-step harness everything on the device is compared with)
against statements that do not share its code: fp64 numpy forms of the reference kernels
(QW/kernels/{rmsnorm,rope,attention,mlp,bias_add,utils}.cl, rotary tables
QW/src/layers/attention.cpp:147-160), closed forms, and probes built so that one plausible
mistake (interleaved instead of half-split rotary pairs, a wrong query-head -> kv-head map, a
dropped eps / scale / max subtraction, keys visited in the wrong order) fails at least one of them.
CPU only."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as O
import decode_harness as DH

L = O.lib
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
I, F32 = C.c_int, C.c_float
for name, args in {
    "orc_rmsnorm": [_u16p, _u16p, _u16p, I, F32],
    "orc_bias_add": [_u16p, _u16p, I],
    "orc_element_add": [_u16p, _u16p, I],
    "orc_rope": [_u16p, I, I, _u16p, _u16p],
    "orc_swiglu": [_u16p, _u16p, I],
    "orc_gqa_attention": [_u16p, _u16p, _u16p, _u16p, _u16p, I, I, I, I, I],
    "orc_rope_tables": [I, I, F32, _u16p, _u16p],
}.items():
    getattr(L, name).restype, getattr(L, name).argtypes = None, args


def h(a):
    """fp16 bits of an array of values (one rounding from fp64)."""
    return np.ascontiguousarray(np.asarray(a, np.float64).astype(np.float16)).view(np.uint16)


def val(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)


def ulp16(x):
    """Spacing of fp16 at |x| (subnormal spacing below 2^-14)."""
    x = np.maximum(np.abs(np.asarray(x, np.float64)), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(x)) - 10)


def assert_within_ulps(got_bits, want, n=1.0):
    got = val(got_bits)
    err = np.abs(got - want)
    lim = n * ulp16(want)
    assert np.all(err <= lim), f"max {np.max(err / ulp16(want)):.2f} fp16 steps at {np.argmax(err / ulp16(want))}"


# ---------------------------------------------------------------- rmsnorm

def rmsnorm64(x, w, eps):
    x, w = val(x), val(w)
    return w * (x / np.sqrt(np.mean(x * x) + eps))


@pytest.mark.parametrize("cols", [4, 64, 70, 252, 256, 576, 896, 1027, 4864])
def test_rmsnorm_against_fp64(cols):
    rng = np.random.default_rng(cols)
    x = h(rng.normal(0, 1.0, cols))
    w = h(1.0 + rng.normal(0, 0.1, cols))
    out = np.empty(cols, np.uint16)
    L.orc_rmsnorm(x, w, out, cols, 1e-6)
    assert_within_ulps(out, rmsnorm64(x, w, 1e-6), 1.0)


def test_rmsnorm_eps_and_mean_are_there():
    # Values of 1e-3: mean(x^2) = 1e-6 = eps, so a dropped eps changes the result by sqrt(2),
    # and a sum in place of the mean by sqrt(cols).
    cols = 896
    x = h(np.full(cols, 1e-3))
    w = h(np.ones(cols))
    out = np.empty(cols, np.uint16)
    L.orc_rmsnorm(x, w, out, cols, 1e-6)
    xv = val(x)[0]
    assert_within_ulps(out, np.full(cols, xv / np.sqrt(xv * xv + 1e-6)), 1.0)
    # scale invariance away from eps: rmsnorm(8 x) = rmsnorm(x), exactly (a power of two)
    rng = np.random.default_rng(1)
    x1 = h(rng.normal(0, 1.0, cols))
    x8 = h(val(x1) * 8.0)
    o1, o8 = np.empty(cols, np.uint16), np.empty(cols, np.uint16)
    L.orc_rmsnorm(x1, w, o1, cols, 0.0)
    L.orc_rmsnorm(x8, w, o8, cols, 0.0)
    assert np.array_equal(o1, o8)


def test_rmsnorm_weight_index():
    # constant x, distinct weights: out[c] = w[c] * sign: a shifted or strided weight index shows
    cols = 576
    x = h(np.full(cols, 2.0))
    wv = (np.arange(cols) % 1000 + 1) / 64.0
    out = np.empty(cols, np.uint16)
    L.orc_rmsnorm(x, h(wv), out, cols, 0.0)
    assert np.array_equal(out, h(wv))       # x / rms = 1 exactly


# ---------------------------------------------------------------- element-wise

def test_bias_add_and_element_add_are_one_fp32_add():
    rng = np.random.default_rng(3)
    n = 4864
    a = h(rng.normal(0, 1, n))
    b = h(rng.normal(0, 0.02, n))
    want = (a.view(np.float16).astype(np.float32) + b.view(np.float16).astype(np.float32)).astype(np.float16).view(np.uint16)
    got = a.copy()
    L.orc_bias_add(got, b, n)
    assert np.array_equal(got, want)
    got = a.copy()
    L.orc_element_add(got, b, n)
    assert np.array_equal(got, want)
    # ties round to even: 2048 + 1 is not an fp16 number, 2048 + 3 rounds up to 2052
    a2, b2 = h([2048.0, 2048.0, 2050.0]), h([1.0, 3.0, 1.0])
    L.orc_element_add(a2, b2, 3)
    assert list(val(a2)) == [2048.0, 2052.0, 2052.0]


def test_swiglu_closed_form():
    rng = np.random.default_rng(4)
    g = np.concatenate([rng.normal(0, 2, 4000), [0.0, -0.0, 30.0, -30.0, 11.0, -11.0, 1e-4, 65504.0 / 4, -20000.0]])
    u = np.concatenate([rng.normal(0, 1, 4000), [3.0, 3.0, 0.5, 0.5, -2.0, 1.0, 7.0, 1.0, 1.0]])
    gb, ub = h(g), h(u)
    gv, uv = val(gb), val(ub)
    with np.errstate(over="ignore"):
        want = gv / (1.0 + np.exp(-gv)) * uv
    got = gb.copy()
    L.orc_swiglu(got, ub, got.size)
    assert_within_ulps(got, want, 1.0)
    # up is the second operand and is not activated: swiglu(g, u) is linear in u (power of two)
    got2 = gb.copy()
    L.orc_swiglu(got2, h(uv * 4.0), got2.size)
    big = np.abs(val(got)) > 2.0 ** -12          # away from subnormals, where x4 is exact
    assert np.array_equal(val(got2)[big], 4.0 * val(got)[big])


# ---------------------------------------------------------------- rotary embedding

@pytest.mark.parametrize("D,theta,max_pos", [(16, 10000.0, 48), (64, 1000000.0, 300), (128, 500000.0, 64)])
def test_rope_tables_against_fp64(D, theta, max_pos):
    cosT = np.empty((max_pos, D), np.uint16)
    sinT = np.empty((max_pos, D), np.uint16)
    L.orc_rope_tables(max_pos, D, theta, cosT, sinT)
    t = np.arange(max_pos, dtype=np.float64)[:, None]
    i = np.arange(D // 2, dtype=np.float64)[None, :]
    ang = t * theta ** (-2.0 * i / D)
    # the reference's fp32 angle carries a relative error of a few 2^-24: |d cos| <= |angle| * 2^-22
    slack = np.abs(ang) * 2.0 ** -22
    for tab, want in ((cosT, np.cos(ang)), (sinT, np.sin(ang))):
        for half in (tab[:, :D // 2], tab[:, D // 2:]):
            assert np.all(np.abs(val(half) - want) <= 0.5 * ulp16(want) * 1.02 + slack)
        assert np.array_equal(tab[:, :D // 2], tab[:, D // 2:])
    assert np.all(val(cosT[0]) == 1.0) and np.all(val(sinT[0]) == 0.0)


def _tables(D, theta, max_pos):
    cosT = np.empty((max_pos, D), np.uint16)
    sinT = np.empty((max_pos, D), np.uint16)
    L.orc_rope_tables(max_pos, D, theta, cosT, sinT)
    return cosT, sinT


def test_rope_position_zero_is_identity():
    D, heads = 64, 5
    cosT, sinT = _tables(D, 1e6, 4)
    x = h(np.random.default_rng(5).normal(0, 1, heads * D))
    y = x.copy()
    L.orc_rope(y, heads, D, cosT[0].copy(), sinT[0].copy())
    assert np.array_equal(x, y)


def test_rope_one_hot_lands_on_its_half_split_partner():
    # e_i (i < D/2) -> cos at i, sin at i + D/2; e_{i+D/2} -> -sin at i, cos at i + D/2
    # (QW/kernels/rope.cl: x1 = buf[hd], x2 = buf[hd + half_dim]).  An interleaved (2i, 2i+1)
    # pairing, a swapped sign or a head stride other than D fails here.
    D, heads, pos = 16, 3, 7
    cosT, sinT = _tables(D, 10000.0, 16)
    c, s = val(cosT[pos]), val(sinT[pos])
    for head in range(heads):
        for i in range(D // 2):
            x = np.zeros(heads * D)
            x[head * D + i] = 1.0
            y = h(x)
            L.orc_rope(y, heads, D, cosT[pos].copy(), sinT[pos].copy())
            want = np.zeros(heads * D)
            want[head * D + i], want[head * D + i + D // 2] = c[i], s[i]
            assert np.array_equal(val(y), want)
            x = np.zeros(heads * D)
            x[head * D + i + D // 2] = 1.0
            y = h(x)
            L.orc_rope(y, heads, D, cosT[pos].copy(), sinT[pos].copy())
            want = np.zeros(heads * D)
            want[head * D + i], want[head * D + i + D // 2] = -s[i], c[i]
            assert np.array_equal(val(y), want)


def test_rope_against_fp64_and_pair_norms():
    D, heads, pos = 64, 14, 37
    cosT, sinT = _tables(D, 1e6, 64)
    rng = np.random.default_rng(6)
    xb = h(rng.normal(0, 1, heads * D))
    y = xb.copy()
    L.orc_rope(y, heads, D, cosT[pos].copy(), sinT[pos].copy())
    x = val(xb).reshape(heads, D)
    c, s = val(cosT[pos])[:D // 2], val(sinT[pos])[:D // 2]
    x1, x2 = x[:, :D // 2], x[:, D // 2:]
    want = np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=1)
    assert_within_ulps(y, want.ravel(), 1.0)
    # a rotation keeps the 2-norm of every (i, i + D/2) pair (to the table's and the store's rounding)
    got = val(y).reshape(heads, D)
    n_in = np.hypot(x1, x2)
    n_out = np.hypot(got[:, :D // 2], got[:, D // 2:])
    assert np.all(np.abs(n_out - n_in) <= 2.0 ** -9 * np.maximum(n_in, 2.0 ** -6))


# ---------------------------------------------------------------- attention

def gqa64(q, kc, vc, n_heads, n_kv, D, seq_k):
    q = val(q).reshape(n_heads, D)
    K = val(kc).reshape(-1, n_kv, D)[:seq_k]
    V = val(vc).reshape(-1, n_kv, D)[:seq_k]
    nrep = n_heads // n_kv
    out = np.zeros((n_heads, D))
    probs = np.zeros((n_heads, seq_k))
    for qh in range(n_heads):
        kvh = qh // nrep
        sc = K[:, kvh, :] @ q[qh] / np.sqrt(D)
        e = np.exp(sc - sc.max())
        p = e / e.sum()
        probs[qh] = p
        out[qh] = p @ V[:, kvh, :]
    return out.ravel(), probs


def run_attention(q, kc, vc, n_heads, n_kv, D, seq_k, stride=None):
    stride = stride or seq_k + 3
    scores = np.zeros(n_heads * stride, np.uint16)
    out = np.zeros(n_heads * D, np.uint16)
    L.orc_gqa_attention(q, kc, vc, scores, out, n_heads, n_kv, D, stride, seq_k)
    return out, scores.reshape(n_heads, stride)[:, :seq_k]


@pytest.mark.parametrize("n_heads,n_kv,D,seq_k", [(4, 2, 16, 9), (14, 2, 64, 38), (9, 3, 64, 1), (6, 6, 32, 20),
                                                  (8, 1, 128, 130), (12, 4, 80, 17)])
def test_attention_against_fp64_gqa(n_heads, n_kv, D, seq_k):
    rng = np.random.default_rng(n_heads * 1000 + seq_k)
    q = h(rng.normal(0, 1.5, n_heads * D))
    kc = h(rng.normal(0, 1.0, (seq_k + 2) * n_kv * D))      # two rows past seq_k that must not be read
    vc = h(rng.normal(0, 1.0, (seq_k + 2) * n_kv * D))
    kc[seq_k * n_kv * D:] = 0x7E00                          # NaN: any use of them poisons the output
    vc[seq_k * n_kv * D:] = 0x7E00
    got, probs = run_attention(q, kc, vc, n_heads, n_kv, D, seq_k)
    want, p64 = gqa64(q, kc, vc, n_heads, n_kv, D, seq_k)
    g = val(got)
    assert np.all(np.isfinite(g))
    # scores, exponentials and probabilities are each stored as fp16 (three roundings of 2^-11)
    assert np.max(np.abs(g - want)) <= 4e-3 * np.max(np.abs(val(vc[:seq_k * n_kv * D])))
    cos = g @ want / (np.linalg.norm(g) * np.linalg.norm(want))
    assert cos >= 0.99999
    assert np.max(np.abs(val(probs) - p64)) <= 2e-3
    assert np.all(np.abs(val(probs).sum(axis=1) - 1.0) <= seq_k * 2.0 ** -12 + 2.0 ** -10)


def test_attention_head_map_and_key_order_probe():
    # V[tk, kvh, :] is the unit vector e_(tk * n_kv + kvh): the output of query head qh then
    # holds its own probabilities p[qh, tk] at element tk * n_kv + (qh // nrep) and zero
    # elsewhere.  qh % n_kv (or any other map), a transposed cache index, or keys in another
    # order put them somewhere else.
    n_heads, n_kv, D, seq_k = 6, 2, 64, 20
    rng = np.random.default_rng(11)
    q = h(rng.normal(0, 2.0, n_heads * D))
    kc = h(rng.normal(0, 1.0, seq_k * n_kv * D))
    V = np.zeros((seq_k, n_kv, D))
    for tk in range(seq_k):
        for kvh in range(n_kv):
            V[tk, kvh, tk * n_kv + kvh] = 1.0
    got, probs = run_attention(q, kc, h(V.ravel()), n_heads, n_kv, D, seq_k)
    g = val(got).reshape(n_heads, D)
    _, p64 = gqa64(q, kc, h(V.ravel()), n_heads, n_kv, D, seq_k)
    nrep = n_heads // n_kv
    for qh in range(n_heads):
        want = np.zeros(D)
        want[np.arange(seq_k) * n_kv + qh // nrep] = val(probs[qh])
        assert np.array_equal(g[qh], want)                  # 1.0 * p summed with zeros: exact
        assert np.max(np.abs(val(probs[qh]) - p64[qh])) <= 1e-3
    # heads of one group see the same keys: distinct q rows give distinct rows of probabilities,
    # but equal q rows in different groups must differ (different K), in the same group must not
    q2 = val(q).reshape(n_heads, D)
    q2[:] = q2[0]
    got2, probs2 = run_attention(h(q2.ravel()), kc, h(V.ravel()), n_heads, n_kv, D, seq_k)
    assert np.array_equal(probs2[0], probs2[1]) and np.array_equal(probs2[0], probs2[2])
    assert np.array_equal(probs2[3], probs2[4]) and not np.array_equal(probs2[0], probs2[3])


def test_attention_large_scores_need_the_max_subtraction_and_the_scale():
    # q.k = 64 * 9 = 576 before scaling; without the 1/sqrt(D) the fp16 score is 576 instead of
    # 72, without the max subtraction exp(72) overflows fp16 storage.
    n_heads, n_kv, D, seq_k = 2, 1, 64, 3
    q = h(np.full(n_heads * D, 3.0))
    K = np.zeros((seq_k, D))
    K[0], K[1], K[2] = 3.0, 3.0 - 8.0 / 64 * 3.0, -3.0       # scores 72, 63, -72
    V = np.zeros((seq_k, D))
    V[0, 0], V[1, 1], V[2, 2] = 1.0, 1.0, 1.0
    got, _ = run_attention(q, h(K.ravel()), h(V.ravel()), n_heads, n_kv, D, seq_k)
    g = val(got).reshape(n_heads, D)
    e = np.exp(np.array([0.0, -9.0, -144.0]))
    p = e / e.sum()
    assert abs(g[0, 0] - p[0]) <= 2.0 ** -11 and abs(g[0, 1] - p[1]) <= 2.0 ** -18 and g[0, 2] == 0.0


# ---------------------------------------------------------------- the whole step

def forward64(model, tokens):
    """Independent fp64 forward of the Qwen2 graph (embedding, [rmsnorm, q/k/v + bias, rotary,
    causal grouped-query attention, o, residual, rmsnorm, silu(gate) * up, down, residual] x L,
    final rmsnorm, lm_head) over the whole token list at once; weights are the dequantised
    int8 rows (q * fp16 scale).  Returns the logits of every position and the last layer's
    q, k (after bias and rotary), v, attention output and silu(gate) * up, per position."""
    c = model.cfg
    Hd, D, nh, nkv = c["hidden"], c["head_dim"], c["n_heads"], c["n_kv_heads"]
    deq = lambda i: model.w8[i].astype(np.float64) * model.ws[i].view(np.float16).astype(np.float64)[:, None]
    f = lambda a: np.asarray(a).view(np.float16).astype(np.float64) if np.asarray(a).dtype == np.uint16 else np.asarray(a, np.float64)
    norm = lambda x, w: f(w) * x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + c["rms_eps"])
    T = len(tokens)
    hcur = f(model.embed)[np.asarray(tokens)]
    pos = np.arange(T)[:, None]
    ang = pos * c["rope_theta"] ** (-2.0 * np.arange(D // 2)[None, :] / D)
    cs, sn = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]

    def rot(x):                                              # [T, heads, D]
        x1, x2 = x[..., :D // 2], x[..., D // 2:]
        return np.concatenate([x1 * cs - x2 * sn, x2 * cs + x1 * sn], axis=-1)

    mask = np.tril(np.ones((T, T), bool))
    for l in range(c["n_layers"]):
        b = 7 * l
        xn = norm(hcur, model.in_norm[l])
        q = rot((xn @ deq(b).T + f(model.bq[l])).reshape(T, nh, D))
        k = rot((xn @ deq(b + 1).T + f(model.bk[l])).reshape(T, nkv, D))
        v = (xn @ deq(b + 2).T + f(model.bv[l])).reshape(T, nkv, D)
        att = np.zeros((T, nh, D))
        for qh in range(nh):
            kvh = qh // (nh // nkv)
            sc = q[:, qh, :] @ k[:, kvh, :].T / np.sqrt(D)
            sc = np.where(mask, sc, -np.inf)
            p = np.exp(sc - sc.max(axis=1, keepdims=True))
            p /= p.sum(axis=1, keepdims=True)
            att[:, qh, :] = p @ v[:, kvh, :]
        hcur = hcur + att.reshape(T, nh * D) @ deq(b + 3).T
        xn = norm(hcur, model.post_norm[l])
        g, u = xn @ deq(b + 4).T, xn @ deq(b + 5).T
        act = g / (1.0 + np.exp(-g)) * u
        hcur = hcur + act @ deq(b + 6).T
    last = dict(q=q.reshape(T, -1), k=k.reshape(T, -1), v=v.reshape(T, -1), att=att.reshape(T, -1), act=act, h=hcur)
    return norm(hcur, model.final_norm) @ deq(7 * c["n_layers"]).T, last


@pytest.mark.parametrize("cfg_name", ["TINY", "GQA3"])
def test_whole_step_against_fp64_forward(cfg_name):
    cfg = DH.TINY if cfg_name == "TINY" else dict(hidden=96, inter=160, n_heads=6, n_kv_heads=2, head_dim=16,
                                                   n_layers=3, vocab=300, max_pos=32, rms_eps=1e-5,
                                                   rope_theta=50000.0)
    model = DH.Model(cfg, seed=77)
    if cfg_name == "GQA3":
        # biases and norm weights large enough that leaving one out moves the logits past the bound
        for l in range(cfg["n_layers"]):
            for b in (model.bq, model.bk, model.bv):
                b[l] = (b[l].astype(np.float32) * 25.0).astype(np.float16)
            model.in_norm[l] = (model.in_norm[l].astype(np.float32) * (1.0 + 0.5 * l)).astype(np.float16)
            model.post_norm[l] = (model.post_norm[l].astype(np.float32) * (2.0 - 0.5 * l)).astype(np.float16)
    cs = model.c_struct()
    dec = DH._lib.orc_decoder_new(C.byref(cs), 1)
    try:
        tokens = [int(t) % cfg["vocab"] for t in DH.PROMPT]
        logits, acts = [], []
        nxt = None
        DH._lib.orc_decoder_buffer.restype = C.c_void_p
        DH._lib.orc_decoder_buffer.argtypes = [C.c_void_p, C.c_int]
        qd, kvd = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
        sizes = dict(h=(0, cfg["hidden"]), q=(1, qd), k=(2, kvd), v=(3, kvd), att=(4, qd), act=(5, cfg["inter"]))
        for pos in range(20):
            if pos >= len(tokens):
                tokens.append(nxt)
            nxt = DH._lib.orc_decoder_step(dec, tokens[pos], pos, None, None, None)
            src = (C.c_uint16 * cfg["vocab"]).from_address(DH._lib.orc_decoder_logits(dec))
            logits.append(np.ctypeslib.as_array(src).copy())
            acts.append({name: np.ctypeslib.as_array((C.c_uint16 * n).from_address(
                DH._lib.orc_decoder_buffer(dec, which))).copy() for name, (which, n) in sizes.items()})
    finally:
        DH._lib.orc_decoder_free(dec)
    want, last = forward64(model, tokens[:20])
    worst_cos, agree = 1.0, 0
    for pos in range(20):
        # the last layer's activations one by one: a missing bias, an unrotated k or a wrong
        # norm weight shows here even where the logits barely move
        for name in sizes:
            g, w = val(acts[pos][name]), last[name][pos]
            assert np.max(np.abs(g - w)) <= 1e-2 * np.max(np.abs(w)) + 1e-4, (name, pos)
        g, w = val(logits[pos]), want[pos]
        worst_cos = min(worst_cos, g @ w / (np.linalg.norm(g) * np.linalg.norm(w)))
        assert np.max(np.abs(g - w)) <= 1e-2 * np.max(np.abs(w)) + 1e-3
        # the greedy token is the fp64 argmax unless the two leading fp64 logits are within rounding
        top = np.argsort(w)[-2:]
        if int(np.argmax(g)) == int(top[1]) or w[top[1]] - w[top[0]] < 2e-3 * np.max(np.abs(w)):
            agree += 1
    assert worst_cos >= 0.9999, worst_cos
    assert agree == 20
