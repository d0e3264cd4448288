"""Quantizers and dequant views of the oracle.

Pins: (1) golden vectors written by the reference's own quantize_row_symmetric /
quantize_row_q4 (tests/golden/make_quantizer_vectors.py); (2) closed forms and
invariants from LF/scripts/quantize_weights.py:53-57 and
LF/scripts/quantize_q4.py:62-82; (3) brute force of the nibble unpack over all
byte values against UNPACK8_FROM_PIXEL (LF/kernels/gemv_m1_q4.cl:31-40)."""
import os

import numpy as np
import pytest

import oracle_lib as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "quantizer_vectors.npz"))


@pytest.mark.parametrize("K", [64, 896])
def test_int8_quantizer_matches_reference_vectors(K):
    w = GOLD[f"int8_w_k{K}"].view(np.float16)
    q, s = O.quantize_int8(w)
    assert np.array_equal(q, GOLD[f"int8_q_k{K}"])
    assert np.array_equal(s, GOLD[f"int8_s_k{K}"])


@pytest.mark.parametrize("K", [64, 896])
def test_q4_quantizer_matches_reference_vectors(K):
    w = GOLD[f"q4_w_k{K}"].view(np.float16)
    p, s = O.quantize_q4(w)
    assert np.array_equal(p, GOLD[f"q4_p_k{K}"])
    assert np.array_equal(s, GOLD[f"q4_s_k{K}"])


def test_int8_quantizer_invariants():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((37, 128)) * 0.02).astype(np.float16)
    w[5] = 0
    q, s = O.quantize_int8(w)
    sf = O.f16(s).astype(np.float64)
    assert q.min() >= -127 and q.max() <= 127
    absmax = np.abs(w.astype(np.float64)).max(axis=1)
    nz = absmax > 0
    assert np.all(np.abs(q[nz]).max(axis=1) == 127)          # the row maximum maps to +-127
    assert np.all(q[5] == 0) and sf[5] == 1.0                 # zero row: scale 1.0, q = 0
    assert np.allclose(sf[nz], absmax[nz] / 127.0, rtol=2**-11)
    # reconstruction error is at most half a step (plus the fp16 rounding of the scale)
    err = np.abs(q * sf[:, None] - w.astype(np.float64))
    assert np.all(err[nz] <= 0.5 * sf[nz, None] * (1 + 2**-9) + 127 * sf[nz, None] * 2**-11)


def test_int8_round_half_to_even():
    # absmax 127 -> scale exactly 1.0 -> q = rint(w): 0.5->0, 1.5->2, 2.5->2, -3.5->-4
    w = np.array([[127.0, 0.5, 1.5, 2.5, -3.5, -0.5, 126.5, -126.5]], np.float16)
    q, s = O.quantize_int8(w)
    assert q.tolist() == [[127, 0, 2, 2, -4, 0, 126, -126]]
    assert O.f16(s)[0] == 1.0


def test_q4_invariants_and_layout():
    rng = np.random.default_rng(4)
    w = (rng.standard_normal((9, 96)) * 0.02).astype(np.float16)
    w[2, 32:64] = 0
    p, s = O.quantize_q4(w)
    assert p.shape == (9, 48) and s.shape == (9, 3)
    lo, hi = p & 15, p >> 4
    stored = np.stack([lo, hi], axis=-1).reshape(9, 96)       # low nibble = even element
    assert stored.min() >= 1 and stored.max() <= 15           # 0 is never produced
    qv = stored.astype(np.int32) - 8
    sf = O.f16(s).astype(np.float64)
    assert np.all(qv[2, 32:64] == 0) and sf[2, 1] == 1.0
    blocks = np.abs(w.astype(np.float64)).reshape(9, 3, 32).max(axis=2)
    nz = blocks > 0
    assert np.all(np.abs(qv).reshape(9, 3, 32).max(axis=2)[nz] == 7)
    assert np.allclose(sf[nz], blocks[nz] / 7.0, rtol=2**-10)
    un = np.empty((9, 96), np.int8)
    O.lib.orc_unpack_q4(p, 9, 96, un)
    assert np.array_equal(un, qv)


def test_q4_rejects_ragged_k():
    w = np.zeros((2, 48), np.uint16)
    assert O.lib.orc_quantize_q4(w, 2, 48, np.zeros((2, 24), np.uint8), np.zeros((2, 2), np.uint16)) == -1


def test_q4_round_half_to_even_and_nibble_order():
    row = np.zeros((1, 32), np.float16)
    row[0, :6] = [7.0, 0.5, 1.5, -2.5, -0.5, 6.5]
    p, s = O.quantize_q4(row)
    assert O.f16(s)[0, 0] == 1.0
    # q = 7,0,2,-2,0,6 -> stored 15,8,10,6,8,14 ; byte i = stored[2i] | stored[2i+1] << 4
    assert p[0, :3].tolist() == [15 | (8 << 4), 10 | (6 << 4), 8 | (14 << 4)]
    assert np.all(p[0, 3:] == (8 | (8 << 4)))


def test_unpack_all_byte_values():
    p = np.arange(256, dtype=np.uint8).reshape(1, 256)
    w = np.empty((1, 512), np.int8)
    O.lib.orc_unpack_q4(p, 1, 512, w)
    for b in range(256):
        assert w[0, 2 * b] == (b & 0xF) - 8
        assert w[0, 2 * b + 1] == ((b >> 4) & 0xF) - 8


def test_dequant_views_index_by_row_and_block():
    # distinct prime-ish values per element make a wrong index visible
    N, K = 5, 64
    q = ((np.arange(N * K).reshape(N, K) * 7) % 255 - 127).astype(np.int8)
    s = np.array([1.0, 0.5, 0.25, 2.0, 0.125], np.float16).view(np.uint16)
    w16 = np.empty((N, K), np.uint16)
    O.lib.orc_dequant_int8_to_f16(q, s, N, K, w16)
    want = (q.astype(np.float32) * O.f16(s).astype(np.float32)[:, None]).astype(np.float16)
    assert np.array_equal(O.f16(w16), want)

    p = ((np.arange(N * K // 2).reshape(N, K // 2) * 37) % 256).astype(np.uint8)
    sc = (2.0 ** -np.arange(N * 2).reshape(N, 2)).astype(np.float16).view(np.uint16)
    wf = np.empty((N, K), np.float32)
    O.lib.orc_dequant_q4_to_f32(p, sc, N, K, wf)
    nib = np.stack([p & 15, p >> 4], -1).reshape(N, K).astype(np.float32) - 8
    want = nib * np.repeat(O.f16(sc).astype(np.float32), 32, axis=1)
    assert np.array_equal(wf, want)
