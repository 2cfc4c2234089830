"""Closed-form and brute-force pins of the packed layout and of the oracle's
arithmetic, independent of the golden vectors."""
import numpy as np
import pytest

from oracle import cherryq_oracle as orc


def test_4bit_all_bytes():
    # every byte value: low nibble is the even position, high nibble the odd one
    q = np.arange(256, dtype=np.uint8).reshape(1, 256)
    u = orc.unpack_codes(q, 4)
    np.testing.assert_array_equal(u[0], np.arange(256) & 15)
    np.testing.assert_array_equal(u[1], np.arange(256) >> 4)
    np.testing.assert_array_equal(orc.pack_codes(u, 4), q)


def test_3bit_all_units_exhaustive():
    # all 2^24 units: three byte rows are the little-endian 24-bit word of eight 3-bit codes
    w24 = np.arange(1 << 24, dtype=np.uint32)
    q = np.stack([(w24 >> (8 * j)) & 0xFF for j in range(3)]).astype(np.uint8)
    u = orc.unpack_codes(q, 3)
    for i in range(8):
        np.testing.assert_array_equal(u[i], (w24 >> (3 * i)) & 7)
    np.testing.assert_array_equal(orc.unpack_codes_kernel_decode(q), u)
    np.testing.assert_array_equal(orc.pack_codes(u, 3), q)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_pack_matches_reference_row_loops(bits):
    rng = np.random.default_rng(bits)
    u = rng.integers(0, 2 ** bits, size=(64, 24), dtype=np.uint8)
    a = orc.pack_codes(u, bits)
    b = orc.pack_codes_reference_loops(u, bits)
    np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(orc.unpack_codes(a, bits), u)


def test_3bit_single_code_positions():
    # code i of a unit set to 7, all others 0: exactly bits 3i..3i+2 of the 24-bit word
    for i in range(8):
        u = np.zeros((8, 1), dtype=np.uint8)
        u[i] = 7
        q = orc.pack_codes(u, 3)[:, 0].astype(np.uint32)
        assert (q[0] | q[1] << 8 | q[2] << 16) == 7 << (3 * i)


@pytest.mark.parametrize("bits", [3, 4])
def test_dequant_value_closed_form(bits):
    # (q + 0.5) * s in fp16 == RN16((u - c_b) * s) computed in float64, for every code
    # and a sweep of every finite positive fp16 scale
    s = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)
    lo, hi = orc.iinfo(bits)
    c_b = 2 ** (bits - 1) - 0.5
    for q in range(lo, hi + 1):
        got = orc.dequantize(np.full(s.shape, q, dtype=np.int8), s)
        with np.errstate(over="ignore"):
            want = ((q - lo - c_b) * s.astype(np.float64)).astype(np.float16)
        np.testing.assert_array_equal(got, want)


def test_quantize_ties_and_clamp():
    # w/s = 3.0 -> 2.5 -> rne 2 ; 4.0 -> 3.5 -> 4 ; +-8 clamp to +-7.99 -> 7 / -8
    s = np.float16(0.125)
    w = (np.array([3.0, 4.0, 8.0, 100.0, -8.0, -100.0, 0.0, -0.5, 0.5]) * 0.125).astype(np.float16)
    q = orc.quantize(w, np.full(w.shape, s), 4)
    np.testing.assert_array_equal(q, [2, 4, 7, 7, -8, -8, 0, -1, 0])


@pytest.mark.parametrize("bits,gs,k,n,frac", [(4, 128, 512, 16, 1 / 32), (3, 128, 512, 16, 1 / 32),
                                              (3, 64, 256, 8, 1 / 16), (4, 128, 2048 + 256, 8, 1 / 256)])
def test_pack_unpack_invariants(bits, gs, k, n, frac):
    w, p = orc.synthetic_layer(k, n, bits, gs, seed=11, cherry_fraction=frac)
    idx = p["cherry_indices"].astype(np.int64)
    dense = orc.unpack(p, bits, gs, k)
    # cherry columns come back exactly
    np.testing.assert_array_equal(dense[:, idx], w[:, idx])
    # normal columns: |w - deq| <= s/2 (+ fp16 rounding of the product), codes in range
    nidx = orc.normal_indices(k, idx)
    s = orc.expand_scales(p["scales"].T, gs, nidx.size).astype(np.float64)
    err = np.abs(w[:, nidx].astype(np.float64) - dense[:, nidx].astype(np.float64))
    assert np.all(err <= s / 2 + np.abs(dense[:, nidx].astype(np.float64)) * 2 ** -10 + 1e-7)
    u = orc.unpack_codes(p["qweight"], bits)
    assert u.max() <= 2 ** bits - 1
    # the max-magnitude element of each group maps to an extreme code
    kn = nidx.size
    for g0 in range(0, kn, gs):
        blk = w[:, nidx[g0:g0 + gs]].astype(np.float32)
        am = np.argmax(np.abs(blk), axis=1)
        codes = u[g0 + am, np.arange(n)]
        assert np.all((codes == 0) | (codes == 2 ** bits - 1))
    # unpack(pack(W)) equals the fake-quantised weight except at rounding ties: quantize()
    # subtracts 0.5 in float32, transform() in fp16 (llama/quantizer.py:158 vs :169), so a
    # handful of elements may land one grid step apart.  Fake quantisation is idempotent.
    adj = orc.adjust_weight(w, idx, bits, gs)
    diff = dense != adj
    assert diff.mean() < 1e-3
    dn, an = dense[:, nidx].astype(np.float64), adj[:, nidx].astype(np.float64)
    assert np.all(np.abs(dn - an) <= s * 1.001)
    np.testing.assert_array_equal(dense[:, idx], adj[:, idx])
    np.testing.assert_array_equal(orc.adjust_weight(adj, idx, bits, gs)[:, idx], adj[:, idx])


@pytest.mark.parametrize("bits", [3, 4])
def test_fused_equals_dense_float64(bits):
    # the entry-point contract (un-rounded weights) against an independent dense float64 product
    k, n, gs = 512, 24, 128
    w, p = orc.synthetic_layer(k, n, bits, gs, seed=5, cherry_fraction=1 / 32)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, k)).astype(np.float16)
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    u = orc.unpack_codes(p["qweight"], bits).astype(np.float64)
    dense = np.zeros((n, k))
    for j, kk in enumerate(nidx):
        dense[:, kk] = (u[j] - (2 ** (bits - 1) - 0.5)) * p["scales"][j // gs].astype(np.float64)
    dense[:, idx] = p["cherry_weight"].T.astype(np.float64)
    want = x.astype(np.float64) @ dense.T
    got = orc.fused_forward(x, p, bits, gs)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
    # one-hot activations read back single dequantised columns
    e = np.zeros((1, k), dtype=np.float16)
    e[0, nidx[200]] = 1
    np.testing.assert_allclose(orc.fused_forward(e, p, bits, gs)[0], dense[:, nidx[200]], rtol=0, atol=0)
    # the CUDA kernels' evaluation order stays within tolerance of it
    ref = orc.fused_reference_order(x, p, bits, gs)
    assert orc.rel_l2(ref, want) <= 2e-3


def test_constant_codes_closed_form():
    # all codes equal u0: y[n] = (u0 - 7.5) * s[n] * sum(x_normal) + cherry term
    k, n, gs, bits = 256, 8, 128, 4
    c = 8
    idx = np.arange(3, 3 + 8 * c, 8)[:c].astype(np.int16)
    kn = k - c
    u = np.full((kn, n), 11, dtype=np.uint8)
    p = {"cherry_indices": idx, "cherry_weight": np.zeros((c, n), np.float16),
         "qweight": orc.pack_codes(u, bits), "scales": np.full((2, n), 0.25, np.float16)}
    x = np.ones((1, k), dtype=np.float16)
    y = orc.fused_forward(x, p, bits, gs)
    np.testing.assert_allclose(y, np.full((1, n), 3.5 * 0.25 * kn))


def test_dequantize_normal_closed_form():
    rng = np.random.default_rng(3)
    for bits in (3, 4):
        kn, n = 240, 8
        u = rng.integers(0, 2 ** bits, size=(kn, n), dtype=np.uint8)
        s = rng.random((2, n), dtype=np.float32)
        out = orc.dequantize_normal(orc.pack_codes(u, bits), s, bits, 256, 16, 128)
        want = (u.astype(np.float32) - (2 ** (bits - 1) - 0.5)) * np.repeat(s, 128, axis=0)[:kn]
        np.testing.assert_array_equal(out, want)
