"""The numpy oracle against vectors recorded from the reference's own Python
(tests/golden/make_golden.py).  Everything here is bit-exact unless stated."""
import glob
import os

import numpy as np
import pytest

from oracle import cherryq_oracle as orc

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "golden_*.npz")))


def load(path):
    d = np.load(path)
    bits, gs, k, n, c = (int(v) for v in d["meta"])
    return d, bits, gs, k, n, c


def test_fixture_set_is_complete():
    assert len(GOLDEN) == 9


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[7:-4] for p in GOLDEN])
class TestGolden:
    def test_schema(self, path):
        d, bits, gs, k, n, c = load(path)
        shapes = orc.buffer_shapes(bits, gs, k, n, float(d["cherry_fraction"][0]))
        assert orc.num_cherries(k, float(d["cherry_fraction"][0])) == c
        for name, (shape, dtype) in shapes.items():
            assert d[name].shape == shape, name
            assert d[name].dtype == dtype, name

    def test_quantizer_functions(self, path):
        d, bits, gs, k, n, c = load(path)
        grp = d["q_group"]
        s = orc.get_scaling_factor(grp, bits)
        assert s.dtype == d["q_scale"].dtype
        np.testing.assert_array_equal(s, d["q_scale"])
        q = orc.quantize(grp, d["q_scale"], bits)
        np.testing.assert_array_equal(q, d["q_quantize"])
        lo, hi = orc.iinfo(bits)
        assert q.min() >= lo and q.max() <= hi
        np.testing.assert_array_equal(orc.dequantize(d["q_quantize"].astype(np.int8), d["q_scale"]),
                                      d["q_dequantize"])
        np.testing.assert_array_equal(orc.transform(grp, d["q_scale"], bits), d["q_transform"])

    def test_scaling_factors_and_adjust_weight(self, path):
        d, bits, gs, k, n, c = load(path)
        g = gs if gs != -1 else k
        idx = np.sort(d["cherry_indices_in"])
        nw = d["weight"][:, orc.normal_indices(k, idx)]
        np.testing.assert_array_equal(orc.get_scaling_factors(nw, bits, g), d["scaling_factors"])
        np.testing.assert_array_equal(orc.adjust_weight(d["weight"], idx, bits, g), d["adjust_weight"])

    def test_pack(self, path):
        d, bits, gs, k, n, c = load(path)
        p = orc.pack(d["weight"], d["cherry_indices_in"], bits, gs)
        for name in ("cherry_indices", "cherry_weight", "qweight", "scales"):
            assert p[name].dtype == d[name].dtype, name
            np.testing.assert_array_equal(p[name], d[name], err_msg=name)

    def test_unpack(self, path):
        d, bits, gs, k, n, c = load(path)
        packed = {name: d[name] for name in ("cherry_indices", "cherry_weight", "qweight", "scales")}
        w = orc.unpack(packed, bits, gs, k)
        assert w.dtype == np.float16
        np.testing.assert_array_equal(w, d["unpack"])

    def test_dequantized_forward(self, path):
        # torch's CPU fp16 linear has an unspecified summation order: tolerance, not bits.
        d, bits, gs, k, n, c = load(path)
        y = orc.dequant_forward(d["x"], d["unpack"])
        assert orc.rel_l2(y, d["forward_dequantized"]) <= 1e-3
        packed = {name: d[name] for name in ("cherry_indices", "cherry_weight", "qweight", "scales")}
        y2 = orc.fused_forward(d["x"], packed, bits, gs)
        assert orc.rel_l2(y2, d["forward_dequantized"]) <= 1e-3

    def test_gather_offset_matches_normal_indices(self, path):
        d, bits, gs, k, n, c = load(path)
        idx = d["cherry_indices"]
        kn = k - c
        ks = np.arange(kn)
        np.testing.assert_array_equal(ks + orc.gather_offset(ks, idx), orc.normal_indices(k, idx))
