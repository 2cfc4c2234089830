"""The fused fake-quantisation kernel (training-side weight of the reference's
llama/cherry_linear.py:77-99) against the recorded vectors and the numpy oracle, bit for bit,
through the C ABI's Python binding (MI355X only)."""
import glob
import os
import sys

import numpy as np
import pytest
import torch

from oracle import cherryq_oracle as orc

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "golden_*.npz")))


@pytest.fixture(scope="module")
def qc():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import quant_cuda
    return quant_cuda


def announce(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def bits_of(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def run(qc, bits, w, idx, g, ste=False):
    wt = torch.from_numpy(np.ascontiguousarray(w)).cuda()
    it = torch.from_numpy(np.asarray(idx, dtype=np.int32)).cuda()
    out = qc.fake_quant_cherryq(bits, wt, it, g, ste=ste)
    torch.cuda.synchronize()
    assert torch.equal(wt.cpu(), torch.from_numpy(np.ascontiguousarray(w)))  # the input is left alone
    return out.cpu().numpy()


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[7:-4] for p in GOLDEN])
def test_recorded_adjust_weight(qc, path):
    """adjust_weight of every fixture (fp16 and fp32 weights), recorded from the reference."""
    d = np.load(path)
    bits, gs, k, n, c = (int(v) for v in d["meta"])
    announce("fake-quant golden", os.path.basename(path))
    g = gs if gs != -1 else k
    got = run(qc, bits, d["weight"], d["cherry_indices_in"], g)
    assert got.dtype == d["adjust_weight"].dtype
    np.testing.assert_array_equal(bits_of(got), bits_of(d["adjust_weight"]))


CASES = [
    # n, k, c, group, bits, dtype, what
    (48, 1024, 8, 128, 4, np.float16, "plain"),
    (48, 1024, 8, 128, 3, np.float32, "plain"),
    (33, 1000, 5, 100, 4, np.float16, "group not a multiple of 8, odd cherry count"),
    (33, 1003, 7, 128, 3, np.float16, "K not a multiple of 8: element-wise path"),
    (17, 1003, 7, 64, 4, np.float32, "K not a multiple of 8: element-wise path"),
    (20, 512, 0, 128, 4, np.float16, "no cherries"),
    (20, 512, 24, 512, 3, np.float32, "one group per row"),
    (20, 512, 24, 3, 2, np.float16, "tiny groups, 2 bits"),
    (9, 4096, 16, 128, 4, np.float32, "wide row"),
    (5, 16384, 64, 128, 3, np.float16, "several chunks per thread"),
    (1500, 256, 8, 128, 4, np.float16, "more rows than workgroups"),
]


@pytest.mark.parametrize("n,k,c,g,bits,dtype,what", CASES, ids=[f"{c[0]}x{c[1]}-c{c[2]}-g{c[3]}-w{c[4]}-{np.dtype(c[5]).name}" for c in CASES])
def test_against_oracle(qc, n, k, c, g, bits, dtype, what):
    announce("fake-quant oracle", n, k, c, g, bits, np.dtype(dtype).name, what)
    rng = np.random.default_rng(1000 * bits + k + c)
    w = (rng.standard_normal((n, k)) * 0.02).astype(dtype)
    w[0, :] = 0                                   # an all-zero row: scale 1e-6 / 2^(b-1)
    w[1, ::3] = np.abs(w[1]).max()                # many elements on the clamp
    w[2, : k // 2] *= dtype(1e-3)                 # tiny values: ratios that round across .5
    idx = rng.choice(k, c, replace=False)         # unsorted on purpose
    want = orc.adjust_weight(w, np.sort(idx), bits, g)
    got = run(qc, bits, w, idx, g)
    np.testing.assert_array_equal(bits_of(got), bits_of(want))
    np.testing.assert_array_equal(bits_of(got[:, idx]), bits_of(w[:, idx]))


def test_duplicate_out_of_range_and_all_cherry_indices(qc):
    announce("fake-quant index handling")
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((12, 256)) * 0.05).astype(np.float16)
    idx = np.array([7, 200, 7, 31, 32, 200, 255, 0], dtype=np.int32)
    want = orc.adjust_weight(w, np.unique(idx), 4, 64)
    np.testing.assert_array_equal(bits_of(run(qc, 4, w, idx, 64)), bits_of(want))
    # entries outside [0, K) are ignored
    np.testing.assert_array_equal(bits_of(run(qc, 4, w, np.concatenate([idx, [-1, 256, 100000]]), 64)), bits_of(want))
    # every channel a cherry: the weight comes back unchanged
    np.testing.assert_array_equal(bits_of(run(qc, 3, w, np.arange(256), 64)), bits_of(w))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_straight_through_form_in_place_and_views(qc, dtype):
    """ste: (q - w) + w evaluated by torch on the kernel's q; in place; a misaligned view."""
    announce("fake-quant ste / in place", np.dtype(dtype).name)
    rng = np.random.default_rng(11)
    n, k, g, bits = 40, 2048, 128, 4
    w = (rng.standard_normal((n, k)) * 0.02).astype(dtype)
    w[3, 5] = -0.0
    idx = np.sort(rng.choice(k, 8, replace=False)).astype(np.int32)
    wt, it = torch.from_numpy(w).cuda(), torch.from_numpy(idx).cuda()
    q = qc.fake_quant_cherryq(bits, wt, it, g)
    ste = qc.fake_quant_cherryq(bits, wt, it, g, ste=True)
    assert torch.equal(ste.view(torch.int16 if dtype == np.float16 else torch.int32),
                       ((q - wt) + wt).view(torch.int16 if dtype == np.float16 else torch.int32))
    # in place
    w2 = wt.clone()
    r = qc.fake_quant_cherryq(bits, w2, it, g, out=w2)
    assert r.data_ptr() == w2.data_ptr() and torch.equal(w2, q)
    # storage offset of one element: rows are no longer 16-byte aligned
    flat = torch.empty(n * k + 1, dtype=wt.dtype, device="cuda")
    flat[1:] = wt.flatten()
    view = flat[1:].view(n, k)
    assert view.data_ptr() % 16 != 0
    assert torch.equal(qc.fake_quant_cherryq(bits, view, it, g), q)
    np.testing.assert_array_equal(bits_of(q.cpu().numpy()), bits_of(orc.adjust_weight(w, idx, bits, g)))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_training_module_uses_the_kernel_and_matches_the_torch_operations(qc, dtype):
    """QuantLinear (training side) on the GPU: fused weight == the module's torch-operation
    branch, forward value and weight gradient included."""
    announce("fake-quant module", dtype)
    from llama.cherry_linear import QuantLinear as TrainLinear
    torch.manual_seed(3)
    k, n = 1024, 96
    lin = TrainLinear(k, n, bias=False, w_bits=3, group_size=128, cherryq=True, cherry_fraction=1 / 64).to(dtype).cuda()
    lin.weight.data.normal_(0, 0.02)
    lin.register_cherry_indices(torch.randperm(k)[:lin.num_cherries])
    lin.train()
    assert lin._fused_fake_quant(lin.weight)
    x = torch.randn(4, k, dtype=dtype, device="cuda")

    def step():
        lin.weight.grad = None
        y = lin(x)
        y.float().square().sum().backward()
        return y.detach().clone(), lin.weight.grad.detach().clone()

    y_fused, g_fused = step()
    w_fused = lin._adjust_weight(lin.weight, ste=False)
    lin._fused_fake_quant = lambda weight: False
    y_torch, g_torch = step()
    w_torch = lin._adjust_weight(lin.weight, ste=False)
    want = orc.adjust_weight(lin.weight.detach().cpu().numpy(), np.sort(lin.cherry_indices.cpu().numpy()), 3, 128)
    np.testing.assert_array_equal(bits_of(w_fused.cpu().numpy()), bits_of(want))
    assert torch.equal(w_fused, w_torch)
    assert torch.equal(y_fused, y_torch)
    assert torch.equal(g_fused, g_torch)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_plain_qat_branch_uses_the_kernel_and_matches_the_torch_operations(qc, dtype):
    """cherryq=False in training mode: whole-row groups through the kernel (no cherry channels)
    against the quantiser's autograd function, value and weight gradient."""
    announce("fake-quant plain QAT", dtype)
    from llama.cherry_linear import QuantLinear as TrainLinear
    torch.manual_seed(5)
    k, n = 1024, 64
    lin = TrainLinear(k, n, bias=False, w_bits=4, group_size=128, cherryq=False).to(dtype).cuda()
    lin.weight.data.normal_(0, 0.02)
    lin.train()
    assert lin._fused_plain(lin.weight)
    x = torch.randn(3, k, dtype=dtype, device="cuda")

    def step():
        lin.weight.grad = None
        y = lin(x)
        y.float().square().sum().backward()
        return y.detach().clone(), lin.weight.grad.detach().clone()

    y_fused, g_fused = step()
    lin._fused_plain = lambda weight: False
    y_torch, g_torch = step()
    assert torch.equal(y_fused, y_torch)
    assert torch.equal(g_fused, g_torch)
    want = orc.adjust_weight(lin.weight.detach().cpu().numpy(), np.empty(0, np.int64), 4, 128)
    got = qc.fake_quant_cherryq(4, lin.weight.detach(), None, 128)
    np.testing.assert_array_equal(bits_of(got.cpu().numpy()), bits_of(want))


@pytest.mark.parametrize("bits", [3, 4])
def test_full_size_layer_against_device_pack_and_unpack(qc, bits):
    """4096 -> 11008 in fp16: the kernel agrees with unpack(pack(w)) (two other kernels) except
    where the fp16 rounding of  w / s - 0.5  crosses a tie, which moves one code by one step."""
    announce("fake-quant full size", bits)
    n, k, g = 11008, 4096, 128
    gen = torch.Generator(device="cuda").manual_seed(bits)
    w = (torch.randn(n, k, device="cuda", generator=gen) * 0.02).half()
    idx = torch.randperm(k, device="cuda", generator=gen)[:16].sort().values
    fq = qc.fake_quant_cherryq(bits, w, idx.int(), g)
    i16, cw, qw, sc = qc.pack_cherryq(bits, w, idx, g)
    dense = qc.unpack_cherryq(bits, qw, cw, i16, sc, k, g)
    assert torch.equal(fq[:, idx], w[:, idx])
    diff = fq != dense
    assert diff.float().mean().item() < 2e-3
    keep = torch.ones(k, dtype=torch.bool, device="cuda")
    keep[idx] = False
    s = sc.t().repeat_interleave(g, dim=1)[:, : k - 16].float()        # (n, Kn)
    err = (fq[:, keep].float() - w[:, keep].float()).abs()
    assert float((err / s).max()) <= 0.52           # half a grid step, plus the fp16 roundings
    step = (fq[:, keep].float() - dense[:, keep].float()).abs()
    assert bool((step <= s * 1.01).all())


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_every_fp16_weight_under_every_fp16_group_maximum(qc, bits):
    """Exhaustive over (group maximum, weight): one row per positive finite fp16 maximum M, holding
    every fp16 bit pattern of magnitude <= M.  The fp16 kernel replaces the division by a
    reciprocal and one correction step; here every quotient it can ever form is compared with
    torch's own fp16 operations on the device, and sampled rows with the numpy oracle."""
    announce("fake-quant exhaustive fp16", bits)
    from llama.quantizer import FullSymQuantizer
    k = 65536
    pats = torch.arange(k, dtype=torch.int32, device="cuda").to(torch.int16)           # every bit pattern
    vals = pats.view(torch.float16)
    mags = (pats.to(torch.int32) & 0x7fff)
    none = torch.empty(0, dtype=torch.int32, device="cuda")
    rng = np.random.default_rng(bits)
    sampled = set(rng.choice(np.arange(1, 0x7c00), 24, replace=False).tolist()) | {1, 2, 0x03ff, 0x0400, 0x7bff}
    for m0 in range(1, 0x7c00, 1024):
        m1 = min(m0 + 1024, 0x7c00)
        mx_pat = torch.arange(m0, m1, dtype=torch.int32, device="cuda")                # (rows,)
        mx = mx_pat.to(torch.int16).view(torch.float16)
        w = torch.where(mags[None, :] <= mx_pat[:, None], vals[None, :], mx[:, None]).contiguous()
        got = qc.fake_quant_cherryq(bits, w, none, k)
        s = FullSymQuantizer.get_scaling_factor(w, None, bits, False)
        want = FullSymQuantizer.transform(w, s, bits)
        same = got.view(torch.int16) == want.view(torch.int16)
        if not bool(same.all()):
            r, c = (~same).nonzero()[0].tolist()
            raise AssertionError(f"max pattern {m0 + r:#x}, weight pattern {c:#x}: kernel "
                                 f"{got[r, c].item()!r}, torch {want[r, c].item()!r}")
        for m in sorted(sampled):
            if m0 <= m < m1:
                row = w[m - m0:m - m0 + 1].cpu().numpy()
                np.testing.assert_array_equal(bits_of(got[m - m0:m - m0 + 1].cpu().numpy()),
                                              bits_of(orc.adjust_weight(row, np.empty(0, np.int64), bits, k)))
        del w, got, s, want, same
