"""Host-side mirror of the reference modules (llama/quantizer.py, llama/cherry_linear.py,
llama/qlinear.py of this package) against the vectors recorded from the reference's Python.
Runs on the CPU; the fused kernels are not involved."""
import glob
import os

import numpy as np
import pytest
import torch

from llama.cherry_linear import QuantLinear as TrainLinear
from llama.qlinear import QuantLinear as PackedLinear, pack_codes, unpack_codes
from llama.quantizer import FullSymQuantizer, RestrictedSymQuantizer

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "golden_*.npz")))
IDS = [os.path.basename(p)[7:-4] for p in GOLDEN]


def build(d):
    bits, gs, k, n, c = (int(v) for v in d["meta"])
    frac = float(d["cherry_fraction"][0])
    w = torch.from_numpy(d["weight"])
    lin = TrainLinear(k, n, bias=False, w_bits=bits, group_size=gs if gs != -1 else k, cherryq=True,
                      cherry_fraction=frac).to(w.dtype)
    lin.weight.data.copy_(w)
    lin.eval()
    lin.register_cherry_indices(torch.from_numpy(d["cherry_indices_in"]))
    q = PackedLinear(bits, gs, lin.quantizer, frac, k, n, bias=False)
    return lin, q, (bits, gs, k, n, c)


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_quantizer_against_reference(path):
    d = np.load(path)
    bits = int(d["meta"][0])
    grp = torch.from_numpy(d["q_group"])
    s = FullSymQuantizer.get_scaling_factor(grp, None, bits, False)
    assert torch.equal(s, torch.from_numpy(d["q_scale"]))
    q = FullSymQuantizer.quantize(grp, s, bits)
    assert q.dtype == torch.int32 and torch.equal(q, torch.from_numpy(d["q_quantize"]))
    assert torch.equal(FullSymQuantizer.dequantize(q.to(torch.int8), s), torch.from_numpy(d["q_dequantize"]))
    assert torch.equal(FullSymQuantizer.transform(grp, s, bits), torch.from_numpy(d["q_transform"]))


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_pack_unpack_forward_against_reference(path):
    d = np.load(path)
    lin, q, (bits, gs, k, n, c) = build(d)
    assert lin.num_cherries == c and q.num_cherries == c
    nw_cols = np.setdiff1d(np.arange(k), d["cherry_indices_in"])
    assert torch.equal(lin._get_scaling_factors(lin.weight[:, torch.from_numpy(nw_cols)]),
                       torch.from_numpy(d["scaling_factors"]))
    assert torch.equal(lin._adjust_weight(lin.weight.clone(), ste=False), torch.from_numpy(d["adjust_weight"]))
    # empty module has the reference's buffer schema
    for name in ("cherry_indices", "cherry_weight", "qweight", "scales"):
        buf = getattr(q, name)
        assert tuple(buf.shape) == d[name].shape and buf.numpy().dtype == d[name].dtype, name
    assert set(q.state_dict().keys()) == {"cherry_indices", "cherry_weight", "qweight", "scales"}
    q.pack(lin)
    for name in ("cherry_indices", "cherry_weight", "qweight", "scales"):
        got = getattr(q, name)
        assert got.device.type == "cpu"
        np.testing.assert_array_equal(got.numpy(), d[name], err_msg=name)
    dense = q.unpack()
    np.testing.assert_array_equal(dense.numpy(), d["unpack"])
    with PackedLinear.dmode(layerwise_dequantize=False):
        y = q(torch.from_numpy(d["x"]))
    assert q.dequantized and not hasattr(q, "scales")
    np.testing.assert_allclose(y.float().numpy(), d["forward_dequantized"].astype(np.float32), rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_code_packing_roundtrip(bits):
    g = torch.Generator().manual_seed(bits)
    codes = torch.randint(0, 2 ** bits, (64, 16), generator=g, dtype=torch.uint8)
    packed = pack_codes(codes, bits)
    assert packed.shape == (64 // 8 * bits, 16) and packed.dtype == torch.uint8
    assert torch.equal(unpack_codes(packed, bits), codes)


def test_dmode_restores_on_exit_and_error():
    assert PackedLinear._layerwise_dequantize is True
    with PackedLinear.dmode(False):
        assert PackedLinear._layerwise_dequantize is False
    assert PackedLinear._layerwise_dequantize is True
    with pytest.raises(ValueError):
        with PackedLinear.dmode(False):
            raise ValueError
    assert PackedLinear._layerwise_dequantize is True


def test_module_surface():
    q = PackedLinear(4, -1, FullSymQuantizer, 1 / 256, 4096, 64, bias=True)
    assert q.group_size == 4096 and q.num_cherries == 16 and q.num_normal == 4080
    assert q.qweight.shape == (2040, 64) and q.scales.shape == (1, 64) and q.bias.shape == (64,)
    q3 = PackedLinear(3, 128, FullSymQuantizer, 1 / 256, 11008, 64, bias=False)
    assert q3.num_cherries == 40 and q3.qweight.shape == (4113, 64) and q3.scales.shape == (86, 64)
    assert q3.bias is None
    with pytest.raises(AssertionError):
        PackedLinear(4, 128, FullSymQuantizer, 1 / 256, 4097, 64)
    t = TrainLinear(256, 8, w_bits=6, group_size=64, cherryq=False)
    assert t.quantizer is RestrictedSymQuantizer
    t5 = TrainLinear(256, 8, w_bits=4, group_size=64, cherryq=True, cherry_fraction=1 / 16)
    assert t5.quantizer is FullSymQuantizer and t5.num_cherries == 16
    assert (t5.cherry_indices == -1).all()


def test_fused_forward_refuses_cpu_tensors():
    q = PackedLinear(4, 128, FullSymQuantizer, 1 / 16, 256, 16, bias=False)
    with pytest.raises(RuntimeError):
        q(torch.zeros(1, 256, dtype=torch.float16))
    q2 = PackedLinear(2, 128, FullSymQuantizer, 1 / 16, 256, 16, bias=False)
    with pytest.raises(NotImplementedError):
        q2(torch.zeros(1, 256, dtype=torch.float16))


def test_training_linear_forward_and_ste():
    torch.manual_seed(0)
    t = TrainLinear(256, 8, w_bits=4, group_size=128, cherryq=True, cherry_fraction=1 / 16)
    t.register_cherry_indices(torch.arange(0, 256, 16))
    x = torch.randn(3, 256)
    t.train()
    y = t(x)
    y.sum().backward()
    assert t.weight.grad is not None and torch.isfinite(t.weight.grad).all()
    # straight-through: d(sum y)/dW = sum_b x[b]
    torch.testing.assert_close(t.weight.grad, x.sum(0).expand(8, 256))
    t.eval()
    w_before = t.weight.detach().clone()
    y2 = t(x)
    assert t.dequantized
    adj = t._adjust_weight(w_before, ste=False)
    torch.testing.assert_close(t.weight.detach(), adj)
    torch.testing.assert_close(y2, torch.nn.functional.linear(x, adj))
