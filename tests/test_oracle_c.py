"""The C oracle against the numpy oracle (which the golden vectors pin) and against
the golden vectors directly."""
import glob
import os

import numpy as np
import pytest

from oracle import cherryq_oracle as orc
from oracle import c_oracle

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "golden_*.npz")))


def test_half_conversions_exhaustive():
    lib = c_oracle.lib()
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    for bits in list(range(0, 65536, 7)) + [0x0001, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0xFBFF, 0x8001]:
        got = lib.cherryq_oracle_h2f(bits)
        want = f[bits]
        assert (np.isnan(want) and np.isnan(got)) or got == want
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 20000),
        (h.view(np.float16).astype(np.float32)[:0x7C00:5]) * np.float32(1 + 2 ** -11),  # exact ties
        (h.view(np.float16).astype(np.float32)[:0x7C00:5]) * np.float32(1 + 2 ** -12),
        np.array([0, 65504, 65519.99, 65520, 1e9, 2 ** -25, 2 ** -24, 3 * 2 ** -26, 2 ** -14], np.float32),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    for v, w in zip(vals.tolist(), want.tolist()):
        assert lib.cherryq_oracle_f2h(v) == w, (v, w)


@pytest.mark.parametrize("path", [p for p in GOLDEN if "_f32" not in p],
                         ids=[os.path.basename(p)[7:-4] for p in GOLDEN if "_f32" not in p])
def test_unpack_against_golden(path):
    d = np.load(path)
    bits, gs, k, n, c = (int(v) for v in d["meta"])
    packed = {name: d[name] for name in ("cherry_indices", "cherry_weight", "qweight", "scales")}
    np.testing.assert_array_equal(c_oracle.unpack(packed, bits, gs, k), d["unpack"])
    y = c_oracle.dequant_matmul(d["x"], packed, bits, gs)
    assert orc.rel_l2(y, d["forward_dequantized"]) <= 1e-3


@pytest.mark.parametrize("bits,gs,k,n,frac", [(4, 128, 1024, 40, 1 / 64), (3, 128, 1024, 40, 1 / 64),
                                              (3, 64, 512, 16, 1 / 32), (4, 256, 1024, 16, 1 / 64)])
def test_c_matches_numpy(bits, gs, k, n, frac):
    w, p = orc.synthetic_layer(k, n, bits, gs, seed=21, cherry_fraction=frac)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, k)).astype(np.float16)
    dense = orc.unpack(p, bits, gs, k)
    np.testing.assert_array_equal(c_oracle.unpack(p, bits, gs, k), dense)
    y, y64 = c_oracle.linear(x, dense, want_f64=True)
    want = x.astype(np.float64) @ dense.astype(np.float64).T
    np.testing.assert_allclose(y64, want, rtol=1e-12, atol=1e-12)
    np.testing.assert_array_equal(y, want.astype(np.float16))
    np.testing.assert_allclose(c_oracle.fused(x, p, bits, gs), orc.fused_forward(x, p, bits, gs),
                               rtol=1e-11, atol=1e-11)
    c = p["cherry_indices"].shape[0]
    s32 = p["scales"].astype(np.float32)
    np.testing.assert_array_equal(c_oracle.dequantize_normal(p["qweight"], s32, bits, k, c, gs),
                                  orc.dequantize_normal(p["qweight"], s32, bits, k, c, gs))
