"""The load-time repacked weight stream (cherryq_prepack_f16 / cherryq_matvec_prepacked_f16) against
the CPU oracle on identical REFERENCE-layout inputs (MI355X only).

The repack is a bijection of the reference buffers: the device stream must equal the oracle's
numpy statement of the layout byte for byte, and unprepack must give the buffers back.  The
matvec over it meets the same bars as the kernels that read the checkpoint layout: rel-L2 <= 1e-3
against the oracle's dequantise-and-matmul, one-hot activations read the dequantised weights
back bit for bit.
"""
import ctypes
import sys

import numpy as np
import pytest
import torch

from oracle import cherryq_oracle as orc
from oracle import c_oracle

pytestmark = pytest.mark.gpu

TOL = 1e-3
NAMES = ("cherry_indices", "cherry_weight", "qweight", "scales")


@pytest.fixture(scope="module")
def qc():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import quant_cuda
    return quant_cuda


def announce(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def dev(p):
    return {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in p.items() if k in NAMES}


def prepack(qc, bits, p, k, gs=128):
    d = dev(p)
    return qc.prepack_cherryq(bits, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], k, gs)


def run(qc, bits, stream, x, n, c, out=None, accumulate=False):
    xt = torch.from_numpy(x).cuda()
    o = torch.full((1, n), float("nan"), dtype=torch.float16, device="cuda") if out is None else torch.from_numpy(out).cuda()
    qc.matvec_prepacked_cherryq(bits, xt, stream, o, x.shape[1], c, accumulate=accumulate)
    torch.cuda.synchronize()
    return o.cpu().numpy()


# shapes: the headline layers, every launch geometry (units per column 32 / 40 / 64 / 86 / 108), ragged
# last unit, N not a multiple of 16, no cherries at all, two cherry MFMA steps (C = 48)
SHAPES = [(4, 4096, 11008), (3, 4096, 11008), (4, 11008, 4096), (3, 11008, 4096), (4, 4096, 4096), (3, 4096, 4096),
          (3, 5120, 5120), (3, 5120, 13824), (3, 13824, 5120), (4, 8192, 8192), (4, 8192, 1024),
          (4, 1024, 264), (3, 1024, 264), (4, 2304, 40), (3, 768, 24),
          # every launch geometry of the kernel with one workgroup per compute unit, both bit widths, with
          # and without tile walking: 257..512 tiles of up to 32 units, 64 / 88 / 128 / 224 units per column
          (4, 2048, 6000), (3, 2048, 6000), (3, 8192, 8192), (3, 8192, 264), (4, 11008, 4608), (3, 11008, 4608),
          (4, 13824, 5120), (4, 16384, 264), (3, 13824, 264), (4, 28672, 264), (3, 28672, 264), (4, 20480, 4352),
          (3, 24576, 4104),
          # the geometries of the LLaMA-13B widths in the other bit width, and the 96-unit one (12 wavefronts on a tile)
          (4, 5120, 5120), (4, 5120, 13824), (3, 12288, 4096), (4, 12288, 4104), (3, 13824, 8200),
          # 769 to 1024 tiles of up to 32 units: three teams per compute unit and the staging wavefronts as a fourth
          (4, 4096, 16384), (3, 4096, 14008), (4, 1024, 12304)]


@pytest.mark.parametrize("bits,k,n", SHAPES)
def test_stream_is_the_oracle_layout_and_unprepack_inverts_it(qc, bits, k, n):
    announce("prepack", bits, k, n)
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=k + n + bits)
    c = p["cherry_indices"].shape[0]
    stream = prepack(qc, bits, p, k)
    torch.cuda.synchronize()
    want = orc.stream_pack(p, bits, 128, k)
    np.testing.assert_array_equal(stream.cpu().numpy(), want)
    back = qc.unprepack_cherryq(bits, stream, k, n, c, 128)
    torch.cuda.synchronize()
    for name, t in zip(NAMES, back):
        np.testing.assert_array_equal(t.cpu().numpy(), p[name], err_msg=name)


@pytest.mark.parametrize("bits,k,n", SHAPES)
def test_prepacked_matvec_against_oracle(qc, bits, k, n):
    announce("prepacked matvec", bits, k, n)
    small = k * n <= 4096 * 4096
    if small:
        _, p = orc.synthetic_layer(k, n, bits, 128, seed=k + n + bits)
    else:
        p = orc.synthetic_packed_fast(k, n, bits, 128, seed=k + n + bits)
    c = p["cherry_indices"].shape[0]
    x = np.random.default_rng(7).standard_normal((1, k)).astype(np.float16)
    y = run(qc, bits, prepack(qc, bits, p, k), x, n, c)
    assert np.isfinite(y).all()
    y_fused = c_oracle.fused(x, p, bits, 128)
    e = orc.rel_l2(y, y_fused)
    print(f"  rel-L2 vs the un-rounded contract {e:.2e}")
    assert e <= TOL
    if small:
        dense = c_oracle.unpack(p, bits, 128, k)
        assert orc.rel_l2(y, c_oracle.linear(x, dense, want_f64=True)[1]) <= TOL
    ulp_ok = np.abs(y.astype(np.float64) - y_fused) <= np.abs(y_fused) * 2 ** -10 + 1e-3
    assert ulp_ok.mean() > 0.999


@pytest.mark.parametrize("bits,k,n", [(4, 4096, 4096), (3, 4096, 4096), (4, 11008, 512), (3, 11008, 512),
                                      (3, 5120, 520), (4, 8192, 264), (3, 13824, 264), (4, 28672, 264), (3, 28672, 264),
                                      (3, 11008, 4608), (4, 16384, 4112), (4, 5120, 8200), (3, 5120, 8200),
                                      (3, 12288, 264), (4, 13824, 8200), (3, 13824, 8200), (3, 4096, 16384), (4, 2048, 14008)])
def test_prepacked_one_hot_reads_back_dequantised_weights(qc, bits, k, n):
    """x = e_j returns column j of the dense weight: decode, gather around the cherry channels and
    the per-unit grid offset are exact.  Positions probe every code slot of a lane's 32 and both
    ends of units, blocks of 512 and the ragged last unit."""
    announce("prepacked one-hot", bits, k, n)
    _, p = orc.synthetic_layer(k, n, bits, 128, seed=5)
    c = p["cherry_indices"].shape[0]
    stream = prepack(qc, bits, p, k)
    dense = c_oracle.unpack(p, bits, 128, k)
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    kn = len(nidx)
    probes = sorted(set([int(nidx[q]) for q in list(range(0, 34)) + [63, 64, 127, 128, 511, 512, 513, kn - 1, kn - 2,
                                                                     kn - 113, kn // 2 + 3, (kn // 128) * 128 - 1,
                                                                     min(kn - 1, (kn // 128) * 128)]]
                        + [int(idx[0]), int(idx[-1]), int(idx[len(idx) // 2])]))
    for j in probes:
        x = np.zeros((1, k), dtype=np.float16)
        x[0, j] = 1
        y = run(qc, bits, stream, x, n, c)
        np.testing.assert_array_equal(y[0], dense[:, j], err_msg=f"column {j}")
    # a single small activation: the exact product rounded once (into the subnormal range)
    x = np.zeros((1, k), dtype=np.float16)
    x[0, probes[5]] = np.float16(2 ** -9)
    y = run(qc, bits, stream, x, n, c)
    np.testing.assert_array_equal(y[0], c_oracle.fused(x, p, bits, 128)[0].astype(np.float16))


def test_prepacked_matches_reference_layout_kernel_accumulate_and_group_256(qc):
    """Same inputs through both paths agree to the last fp16 bit almost everywhere (both round one
    fp32 sum); accumulate adds into `out`; a group size of 256 is two units per scale row."""
    bits, k, n = 4, 4096, 1024
    _, p = orc.synthetic_layer(k, n, bits, 256, seed=9)
    c = p["cherry_indices"].shape[0]
    d = dev(p)
    x = np.random.default_rng(3).standard_normal((1, k)).astype(np.float16)
    stream = qc.prepack_cherryq(bits, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], k, 256)
    back = qc.unprepack_cherryq(bits, stream, k, n, c, 256)
    np.testing.assert_array_equal(back[3].cpu().numpy(), p["scales"])
    y = run(qc, bits, stream, x, n, c)
    ref = torch.zeros(1, n, dtype=torch.float16, device="cuda")
    qc.matmul_cherryq(bits, torch.from_numpy(x).cuda(), d["qweight"], d["cherry_weight"], d["cherry_indices"],
                      d["scales"], ref, 256, accumulate=False)
    torch.cuda.synchronize()
    r = ref.cpu().numpy()
    assert (y == r).mean() > 0.9 and orc.rel_l2(y, r) < 3e-4  # different summation orders: the last bit may differ
    assert orc.rel_l2(y, c_oracle.fused(x, p, bits, 256)) <= TOL
    base = np.random.default_rng(4).standard_normal((1, n)).astype(np.float16)
    y2 = run(qc, bits, stream, x, n, c, out=base.copy(), accumulate=True)
    want = (c_oracle.fused(x, p, bits, 256) + base.astype(np.float64)).astype(np.float16)
    assert orc.rel_l2(y2, want) <= TOL
    # run-to-run identical (no atomics anywhere in this path)
    np.testing.assert_array_equal(run(qc, bits, stream, x, n, c), y)


def test_prepacked_linearity_at_full_size(qc):
    """4096 -> 11008, both bit widths: f(2 x) == 2 f(x) exactly (powers of two commute with every
    rounding involved) and a column sample against the C oracle."""
    for bits in (4, 3):
        k, n = 4096, 11008
        p = orc.synthetic_packed_fast(k, n, bits, 128, seed=3)
        c = p["cherry_indices"].shape[0]
        stream = prepack(qc, bits, p, k)
        rng = np.random.default_rng(11)
        x1 = rng.standard_normal((1, k)).astype(np.float16)
        y1 = run(qc, bits, stream, x1, n, c)
        y2 = run(qc, bits, stream, (x1 * np.float16(2)).astype(np.float16), n, c)
        np.testing.assert_array_equal(y2, (y1.astype(np.float32) * 2).astype(np.float16))


def test_quantlinear_prepack_forward_and_release(qc):
    from llama.qlinear import QuantLinear
    from llama.quantizer import FullSymQuantizer
    for bits in (4, 3):
        k, n = 4096, 1024
        _, p = orc.synthetic_layer(k, n, bits, 128, seed=21 + bits)
        m = QuantLinear(bits, 128, FullSymQuantizer, 1 / 256, k, n, bias=False)
        for name in NAMES:
            setattr(m, name, torch.from_numpy(p[name]))
        m = m.cuda()
        x = torch.from_numpy(np.random.default_rng(5).standard_normal((1, 1, k)).astype(np.float16)).cuda()
        y0 = m(x)
        assert m.prepack()
        y1 = m(x)
        want = c_oracle.fused(x.reshape(1, k).cpu().numpy(), p, bits, 128)
        assert orc.rel_l2(y1.reshape(1, n).cpu().numpy(), want) <= TOL
        assert orc.rel_l2(y1.cpu().numpy(), y0.cpu().numpy()) < 3e-4
        # other batch sizes keep using the checkpoint-layout kernels
        xb = torch.from_numpy(np.random.default_rng(6).standard_normal((3, k)).astype(np.float16)).cuda()
        assert m(xb).shape == (3, n)
        # release the checkpoint-layout buffers, then bring them back bit for bit
        assert m.prepack(release_reference=True)
        assert m.qweight.numel() == 0
        y2 = m(x)
        assert torch.equal(y1, y2)
        assert orc.rel_l2(m(xb).float().cpu().numpy(), c_oracle.fused(xb.cpu().numpy(), p, bits, 128)) <= TOL
        m.unprepack()
        for name in NAMES:
            np.testing.assert_array_equal(getattr(m, name).cpu().numpy(), p[name], err_msg=name)
        assert m(xb).shape == (3, n)


def test_prepacked_c_abi_rejections(qc):
    lib = qc._lib
    assert lib.cherryq_prepack_bytes(5, 4096, 4096, 16) == 0
    assert lib.cherryq_prepack_supported(4, 2, 4096, 4096, 16, 128) == 1      # 2 to 16 rows: the rows kernel
    assert lib.cherryq_prepack_supported(4, 17, 4096, 4096, 16, 128) == 0
    assert lib.cherryq_prepack_supported(4, 16, 8192, 8192, 32, 128) == 1     # rows kept in registers
    assert lib.cherryq_prepack_supported(3, 2, 13824, 5120, 48, 128) == 1     # more than 64 units per column: in slices
    assert lib.cherryq_prepack_supported(4, 1, 4096, 4096, 16, 64) == 0       # group size a multiple of 128
    assert lib.cherryq_prepack_supported(4, 1, 28672, 8192, 112, 128) == 1    # 224 units per column: the deepest taken
    assert lib.cherryq_prepack_supported(4, 1, 32768, 8192, 128, 128) == 0    # more than 224 units
    assert lib.cherryq_prepack_supported(4, 16, 28672, 8192, 112, 128) == 1   # 2 to 16 rows: four slices of 56 units
    assert lib.cherryq_prepack_supported(3, 1, 13824, 5120, 48, 128) == 1
    nbytes = lib.cherryq_prepack_bytes(4, 4096, 1024, 16)
    buf = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    x = torch.zeros(1, 4096, dtype=torch.float16, device="cuda")
    y = torch.zeros(1, 1024, dtype=torch.float16, device="cuda")
    f = lib.cherryq_matvec_prepacked_f16
    assert f(4, x.data_ptr(), buf.data_ptr(), nbytes - 1, y.data_ptr(), 1, 4096, 1024, 16, 0, None) == -4
    assert f(4, x.data_ptr(), buf.data_ptr(), nbytes, y.data_ptr(), 2, 4096, 1024, 16, 0, None) == -7
    assert f(4, x.data_ptr(), buf.data_ptr(), nbytes, y.data_ptr(), 0, 4096, 1024, 16, 0, None) == 0
    assert f(4, None, buf.data_ptr(), nbytes, y.data_ptr(), 1, 4096, 1024, 16, 0, None) == -1
    assert f(4, x.data_ptr() + 2, buf.data_ptr(), nbytes, y.data_ptr(), 1, 4096, 1024, 16, 0, None) == -6
    assert lib.cherryq_prepack_supported(4, 1, 4096, 8 * 1000 * 1000, 16, 128) == 0  # a stream of 2 GiB and more
    assert f(2, x.data_ptr(), buf.data_ptr(), nbytes, y.data_ptr(), 1, 4096, 1024, 16, 0, None) == -5
    # the entry point for 2 to 16 rows: needs its scratch buffer
    lib.cherryq_prepacked_scratch_bytes.restype = ctypes.c_size_t
    g = lib.cherryq_matmul_prepacked_f16
    x4 = torch.zeros(12, 4096, dtype=torch.float16, device="cuda")
    y4 = torch.zeros(12, 1024, dtype=torch.float16, device="cuda")
    need = lib.cherryq_prepacked_scratch_bytes(4, 12, 4096, 1024, 16)
    assert need >= 12 * 4096 * 2 and lib.cherryq_prepacked_scratch_bytes(4, 1, 4096, 1024, 16) == 0
    sc = torch.empty(need, dtype=torch.uint8, device="cuda")
    assert g(4, x4.data_ptr(), buf.data_ptr(), nbytes, y4.data_ptr(), 12, 4096, 1024, 16, 0, None, 0, None) == -4
    assert g(4, x4.data_ptr(), buf.data_ptr(), nbytes, y4.data_ptr(), 12, 4096, 1024, 16, 0, sc.data_ptr(), need - 1, None) == -4
    assert g(4, x4.data_ptr(), buf.data_ptr(), nbytes, y4.data_ptr(), 17, 4096, 1024, 16, 0, sc.data_ptr(), need, None) == -7
    assert g(4, x4.data_ptr(), buf.data_ptr(), nbytes, y4.data_ptr(), 12, 4096, 1024, 16, 0, sc.data_ptr(), need, None) == 0
    assert g(4, x4.data_ptr() + 2, buf.data_ptr(), nbytes, y4.data_ptr(), 11, 4096, 1024, 16, 0, sc.data_ptr(), need, None) == -6
    # two to eight rows on this layer run in one launch: no scratch buffer
    for rows in (2, 4, 8):
        assert lib.cherryq_prepacked_scratch_bytes(4, rows, 4096, 1024, 16) == 0
        assert g(4, x4.data_ptr(), buf.data_ptr(), nbytes, y4.data_ptr(), rows, 4096, 1024, 16, 0, None, 0, None) == 0
    assert g(4, x4.data_ptr() + 2, buf.data_ptr(), nbytes, y4.data_ptr(), 3, 4096, 1024, 16, 0, None, 0, None) == -6
    assert g(4, x.data_ptr(), buf.data_ptr(), nbytes, y.data_ptr(), 1, 4096, 1024, 16, 0, None, 0, None) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("bits", [4, 3])
@pytest.mark.parametrize("case", ["qkv_norm", "gate_up_norm", "o_accumulate", "qkv_plain"])
def test_prepacked_group_llama7b_shapes_against_the_c_oracle(bits, case):
    """The grouped launch over repacked layers at the decoder's shapes -- 3 x (4096 -> 4096) and
    2 x (4096 -> 11008) behind the fused RMSNorm, 4096 -> 4096 accumulating into the output -- against
    the C oracle's fused product of the prologue's result, and bit for bit on activations whose
    normalised form is one-hot."""
    import cherryq_decoder as dec
    print("[case] prepacked group", bits, case, flush=True)
    K, widths = {"qkv_norm": (4096, (4096, 4096, 4096)), "gate_up_norm": (4096, (11008, 11008)),
                 "o_accumulate": (4096, (4096,)), "qkv_plain": (4096, (4096, 1024, 1024))}[case]
    gen = torch.Generator(device="cuda").manual_seed(23 + bits)
    cfg = dec.DecoderConfig(w_bits=bits, group_size=128, cherry_fraction=1 / 256)
    mods = [dec.random_packed_linear(cfg, K, n, gen, "cuda") for n in widths]
    for m in mods:
        assert m.prepack()
    packed = [{b: getattr(m, b).cpu().numpy() for b in ("qweight", "scales", "cherry_weight", "cherry_indices")} for m in mods]
    f16 = lambda a: np.asarray(a).astype(np.float16)
    rng = np.random.default_rng(9)

    def run(vec, base=None, **kw):
        outs = [torch.full((1, n), 7.0, dtype=torch.float16, device="cuda") if base is None else
                torch.from_numpy(base[i]).cuda() for i, n in enumerate(widths)]
        dec.matvec_group_prepacked(mods, torch.from_numpy(vec).cuda(), outs, **kw)
        torch.cuda.synchronize()
        return [o.cpu().numpy() for o in outs]

    if case.endswith("norm"):
        eps = 1e-6
        h = f16(rng.standard_normal((1, K)) * 3)
        nw = f16(rng.random(K) + 0.5)
        hf = h.astype(np.float64)
        act = f16(nw.astype(np.float64) * f16(hf / np.sqrt(np.mean(hf * hf) + eps)).astype(np.float64))
        got = run(h, norm_weight=torch.from_numpy(nw).cuda(), eps=eps)
        for o, p in zip(got, packed):
            assert orc.rel_l2(o, c_oracle.fused(act, p, bits, 128)) <= 1e-3
        # and the launch over the checkpoint layout with the same prologue agrees
        outs = [torch.empty(1, n, dtype=torch.float16, device="cuda") for n in widths]
        dec.matvec_group(mods, torch.from_numpy(h).cuda(), outs, norm_weight=torch.from_numpy(nw).cuda(), eps=eps)
        torch.cuda.synchronize()
        for o, r in zip(got, outs):
            assert orc.rel_l2(o, r.cpu().numpy().astype(np.float64)) <= 5e-4
        # one-hot through the norm: mean(x^2) + eps = 1 for x = e_j and eps = 1 - 1/K
        nw2 = f16(2.0 ** rng.integers(-2, 3, K))
        for j in (0, 1, 127, 128, 2049, K - 1, int(packed[0]["cherry_indices"][0]), int(packed[-1]["cherry_indices"][-1])):
            x = np.zeros((1, K), dtype=np.float16)
            x[0, j] = 1
            got = run(x, norm_weight=torch.from_numpy(nw2).cuda(), eps=1.0 - 1.0 / K)
            xa = np.zeros((1, K), dtype=np.float16)
            xa[0, j] = nw2[j]
            for o, p in zip(got, packed):
                with np.errstate(over="ignore"):
                    np.testing.assert_array_equal(o[0], f16(c_oracle.fused(xa, p, bits, 128)[0]), err_msg=f"column {j}")
    else:
        x = f16(rng.standard_normal((1, K)))
        acc = case == "o_accumulate"
        base = [f16(rng.standard_normal((1, n))) for n in widths] if acc else None
        got = run(x, base=base, accumulate=acc)
        for i, (o, p) in enumerate(zip(got, packed)):
            want = c_oracle.fused(x, p, bits, 128) + (base[i].astype(np.float64) if acc else 0.0)
            assert orc.rel_l2(o, want) <= 1e-3
        for j in (0, 129, K - 1, int(packed[0]["cherry_indices"][3])):
            e = np.zeros((1, K), dtype=np.float16)
            e[0, j] = 1
            got = run(e, base=base, accumulate=acc)
            for i, (o, p) in enumerate(zip(got, packed)):
                want = c_oracle.fused(e, p, bits, 128) + (base[i].astype(np.float64) if acc else 0.0)
                np.testing.assert_array_equal(o, f16(want), err_msg=f"column {j} member {i}")


def test_prepacked_group_rejections():
    import cherryq_decoder as dec
    lib = dec._lib
    fake = 1 << 12
    one = (dec._StreamLayer * 1)(dec._StreamLayer(fake, 1 << 30, fake, 4096))
    four = (dec._StreamLayer * 4)(*[dec._StreamLayer(fake, 1 << 30, fake, 4096)] * 4)
    f = lib.cherryq_decode_matvec_group_prepacked_f16
    assert f(5, fake, None, 0.0, one, 1, 4096, 16, 0, None) == -5
    assert f(4, None, None, 0.0, one, 1, 4096, 16, 0, None) == -1
    assert f(4, fake, None, 0.0, four, 4, 4096, 16, 0, None) == -2
    assert f(4, fake + 2, None, 0.0, one, 1, 4096, 16, 0, None) == -6
    small = (dec._StreamLayer * 1)(dec._StreamLayer(fake, 64, fake, 4096))
    assert f(4, fake, None, 0.0, small, 1, 4096, 16, 0, None) == -4
    assert f(4, fake, None, 0.0, one, 1, 65536, 0, 0, None) == -7


@pytest.mark.parametrize("bits,k,n", [(4, 4096, 32000), (3, 4096, 32008), (4, 1024, 100000), (3, 2048, 65544)])
def test_prepacked_layers_with_more_tiles_than_resident_workgroups(bits, k, n):
    """Wide layers: a workgroup walks several tiles (activations staged once, the load ring running
    across tile boundaries).  Against the C oracle, one-hot bit for bit (first / last tile, tiles
    taken second and last by a workgroup), accumulate, and repeatable."""
    import quant_cuda
    print("[case] prepacked wide layer", bits, k, n, flush=True)
    p = orc.synthetic_layer(k, n, bits, 128, seed=60 + bits)[1]
    t = {name: torch.from_numpy(np.ascontiguousarray(v)).cuda() for name, v in p.items()
         if name in ("qweight", "scales", "cherry_weight", "cherry_indices")}
    c = int(p["cherry_indices"].shape[0])
    stream = quant_cuda.prepack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"], t["scales"], k, 128)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, k)).astype(np.float16)

    def run(xv, base=None):
        out = torch.full((1, n), 5.0, dtype=torch.float16, device="cuda") if base is None else torch.from_numpy(base).cuda()
        quant_cuda.matvec_prepacked_cherryq(bits, torch.from_numpy(xv).cuda(), stream, out, k, c, accumulate=base is not None)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    want = c_oracle.fused(x, p, bits, 128)
    got = run(x)
    assert orc.rel_l2(got, want) <= 1e-3
    np.testing.assert_array_equal(got, run(x))
    base = rng.standard_normal((1, n)).astype(np.float16)
    assert orc.rel_l2(run(x, base), want + base.astype(np.float64)) <= 1e-3
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    probes = [int(nidx[0]), int(nidx[129]), int(nidx[-1])] + ([int(idx[0]), int(idx[-1])] if len(idx) else [])
    for j in probes:
        e = np.zeros((1, k), dtype=np.float16)
        e[0, j] = 1
        np.testing.assert_array_equal(run(e), c_oracle.fused(e, p, bits, 128).astype(np.float16), err_msg=f"column {j}")


@pytest.mark.parametrize("bits,k,n,b", [(4, 4096, 11008, 16), (3, 4096, 11008, 16), (4, 4096, 4096, 8), (3, 4096, 4096, 2),
                                        (4, 8192, 1024, 8), (3, 1160, 264, 5), (4, 4096, 32008, 13), (4, 1024, 520, 16),
                                        (4, 8192, 4096, 16), (3, 8192, 1032, 9), (4, 4096, 4096, 3),
                                        (3, 4096, 4112, 8), (4, 2048, 16, 16), (3, 1160, 264, 12), (4, 8192, 8200, 16),
                                        # deeper than 64 units: slices of units with fp32 partial outputs and a summing launch
                                        (4, 11008, 4096, 16), (3, 11008, 4096, 2), (3, 13824, 5120, 8), (4, 13824, 264, 11),
                                        (4, 28672, 1032, 16), (3, 28672, 8192, 4), (4, 8320, 528, 5), (3, 16512, 4112, 16),
                                        # two to four rows on every geometry of the one-workgroup-per-compute-unit kernel
                                        (4, 4096, 11008, 4), (3, 4096, 11008, 3), (4, 4096, 8200, 2), (3, 4096, 32008, 4),
                                        (4, 5120, 5120, 4), (3, 5120, 13824, 4), (4, 6144, 12304, 3), (3, 8192, 8192, 4),
                                        (4, 8192, 12304, 2), (4, 11008, 4096, 4), (3, 11008, 4096, 3), (4, 12288, 4096, 4),
                                        (3, 12288, 1032, 2), (4, 1160, 264, 4), (3, 2048, 16, 2), (4, 8192, 1024, 3),
                                        # five to eight rows in the same kernel (layers of up to 48 units)
                                        (4, 4096, 11008, 8), (3, 4096, 11008, 5), (4, 4096, 4096, 7), (3, 4096, 8200, 6),
                                        (4, 5120, 5120, 8), (3, 5120, 13824, 8), (3, 6144, 12304, 7), (4, 1160, 264, 6),
                                        (4, 4096, 32008, 8),
                                        # fewer units per column than a team has wavefronts
                                        (4, 392, 24, 3), (3, 136, 8, 8), (4, 520, 40, 16)])
def test_prepacked_rows_against_the_c_oracle(bits, k, n, b):
    """2 to 16 activation rows over the repacked stream (compaction launch + matrix-core launch with
    real rows): against the C oracle, one-hot rows bit for bit (also with rows of very different
    power-of-two magnitude), accumulate, repeatable, and agreeing with the checkpoint-layout path."""
    import quant_cuda
    print("[case] prepacked rows", bits, k, n, b, flush=True)
    p = orc.synthetic_layer(k, n, bits, 128, seed=70 + bits)[1]
    t = {name: torch.from_numpy(np.ascontiguousarray(v)).cuda() for name, v in p.items()
         if name in ("qweight", "scales", "cherry_weight", "cherry_indices")}
    c = int(p["cherry_indices"].shape[0])
    assert quant_cuda.prepack_supported(bits, b, k, n, c, 128)
    stream = quant_cuda.prepack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"], t["scales"], k, 128)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((b, k)).astype(np.float16)

    def run(xv, base=None):
        out = torch.full((xv.shape[0], n), 5.0, dtype=torch.float16, device="cuda") if base is None else torch.from_numpy(base).cuda()
        quant_cuda.matvec_prepacked_cherryq(bits, torch.from_numpy(xv).cuda(), stream, out, k, c, accumulate=base is not None)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    want = c_oracle.fused(x, p, bits, 128)
    got = run(x)
    for r in range(b):
        assert orc.rel_l2(got[r], want[r]) <= 1e-3, r
    np.testing.assert_array_equal(got, run(x))
    base = rng.standard_normal((b, n)).astype(np.float16)
    acc = run(x, base)
    for r in range(b):
        assert orc.rel_l2(acc[r], want[r] + base[r].astype(np.float64)) <= 1e-3, r
    ref = torch.empty(b, n, dtype=torch.float16, device="cuda")
    quant_cuda.matmul_cherryq(bits, torch.from_numpy(x).cuda(), t["qweight"], t["cherry_weight"], t["cherry_indices"],
                              t["scales"], ref, 128)
    torch.cuda.synchronize()
    assert orc.rel_l2(got, ref.cpu().numpy().astype(np.float64)) <= 5e-4
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    pool = [int(nidx[0]), int(nidx[1]), int(nidx[31]), int(nidx[32]), int(nidx[127]), int(nidx[128]), int(nidx[-1]),
            int(nidx[-33])] + ([int(idx[0]), int(idx[-1]), int(idx[len(idx) // 2])] if len(idx) else [])
    e = np.zeros((b, k), dtype=np.float16)
    for r in range(b):
        e[r, pool[r % len(pool)]] = np.float16(2.0 ** ((r * 5) % 13 - 6))
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(run(e), c_oracle.fused(e, p, bits, 128).astype(np.float16))


def test_prepacked_rows_on_random_small_layers(qc):
    """1 to 16 rows over randomly drawn small layers -- input widths that are no multiple of 512,
    0 to 128 cherry channels at random places (neighbours, the first and the last columns), widths
    that end inside a tile -- against the C oracle, and one-hot rows bit for bit."""
    rng = np.random.default_rng(2024)
    done = 0
    for case in range(60):
        bits = int(rng.choice([3, 4]))
        c = int(rng.choice([0, 8, 16, 24, 40, 64, 96, 128]))
        k = int(rng.integers(17 + c // 8, 420)) * 8
        n = int(rng.integers(1, 90)) * 8
        b = int(rng.integers(1, 17))
        if k - c < 8:
            continue
        frac = (c + 0.5) / k if c else 1e-9
        p = orc.synthetic_packed_fast(k, n, bits, 128, seed=1000 + case, cherry_fraction=frac)
        if p["cherry_indices"].shape[0] != c or not qc.prepack_supported(bits, b, k, n, c, 128):
            continue
        if c and case % 3 == 0:   # neighbours at both ends of the row
            idx = np.sort(np.unique(np.concatenate([np.arange(min(4, c)), k - 1 - np.arange(min(3, c)),
                                                    p["cherry_indices"].astype(np.int64)]))[:c]).astype(np.int16)
            if idx.shape[0] == c:
                p["cherry_indices"] = idx
        announce("random small layer", bits, k, n, c, b)
        stream = prepack(qc, bits, p, k)
        x = rng.standard_normal((b, k)).astype(np.float16)
        out = torch.full((b, n), float("nan"), dtype=torch.float16, device="cuda")
        qc.matvec_prepacked_cherryq(bits, torch.from_numpy(x).cuda(), stream, out, k, c)
        torch.cuda.synchronize()
        got, want = out.cpu().numpy(), c_oracle.fused(x, p, bits, 128)
        for r in range(b):
            assert orc.rel_l2(got[r], want[r]) <= TOL, (case, bits, k, n, c, b, r)
        e = np.zeros((b, k), dtype=np.float16)
        for r in range(b):
            e[r, int(rng.integers(0, k))] = np.float16(2.0 ** int(rng.integers(-4, 4)))
        qc.matvec_prepacked_cherryq(bits, torch.from_numpy(e).cuda(), stream, out, k, c)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.cpu().numpy(), c_oracle.fused(e, p, bits, 128).astype(np.float16),
                                      err_msg=str((case, bits, k, n, c, b)))
        done += 1
    assert done >= 30, done


def test_quantlinear_routes_rows_to_the_stream_after_prepack():
    """QuantLinear.forward after prepack(): 1 to 16 rows run over the weight stream (also with the
    checkpoint-layout buffers released), 17 rows on the checkpoint layout; all agree with the
    module before prepack()."""
    from llama.qlinear import QuantLinear
    from llama.quantizer import FullSymQuantizer
    import cherryq_decoder as dec
    import quant_cuda
    print("[case] QuantLinear rows routing", flush=True)
    cfg = dec.DecoderConfig(w_bits=4, group_size=128, cherry_fraction=1 / 256)
    m = dec.random_packed_linear(cfg, 4096, 1024, torch.Generator(device="cuda").manual_seed(2), "cuda")
    xs = {b: torch.randn(b, 4096, device="cuda", generator=torch.Generator(device="cuda").manual_seed(b)).half()
          for b in (1, 2, 3, 4, 9, 16, 17)}
    before = {b: m(x) for b, x in xs.items()}
    assert m.prepack()
    for b, x in xs.items():
        got = m(x)
        assert got.shape == (b, 1024)
        assert orc.rel_l2(got.float().cpu().numpy(), before[b].float().cpu().numpy().astype(np.float64)) <= 5e-4, b
        if b == 17:
            assert torch.equal(got, before[b]), b   # same kernel as before
        else:
            assert quant_cuda.prepacked_rows_recommended(4, b, 4096, 1024, m.num_cherries, 128), b
    m.prepack(release_reference=True)
    # only the stream is left: every batch size runs over it (2 and 3 rows on the rows kernel,
    # more than 16 in pieces of 16)
    for b in xs:
        assert orc.rel_l2(m(xs[b]).float().cpu().numpy(), before[b].float().cpu().numpy().astype(np.float64)) <= 5e-4, b
    with pytest.raises(RuntimeError):
        m.state_dict()
    with pytest.raises(RuntimeError):
        m.cpu()
    m.unprepack()
    assert torch.equal(m(xs[2]), before[2])
    assert set(m.state_dict()) >= {"qweight", "scales", "cherry_weight", "cherry_indices"}
    # new weights drop a stream made from the old ones
    assert m.prepack()
    other = dec.random_packed_linear(cfg, 4096, 1024, torch.Generator(device="cuda").manual_seed(3), "cuda")
    m.load_state_dict(other.state_dict())
    assert m._stream is None
    assert torch.equal(m(xs[1]), other(xs[1]))
    assert m.prepack()
    m.cpu()
    assert m._stream is None and not m.qweight.is_cuda


def test_quantlinear_deep_layer_rows_after_prepack():
    """A layer deeper than 64 units (11008 input channels) after prepack(): 2 to 4 rows take the
    four-row form of the one-row kernel, 8 to 16 rows leave the checkpoint-layout batch kernel for
    the stream in slices, 5 and 19 stay; with the checkpoint buffers released every batch size runs
    over the stream.  All agree with the module before prepack()."""
    import cherryq_decoder as dec
    print("[case] QuantLinear deep rows routing", flush=True)
    cfg = dec.DecoderConfig(w_bits=3, group_size=128, cherry_fraction=1 / 256)
    m = dec.random_packed_linear(cfg, 11008, 1032, torch.Generator(device="cuda").manual_seed(5), "cuda")
    xs = {b: torch.randn(b, 11008, device="cuda", generator=torch.Generator(device="cuda").manual_seed(b)).half()
          for b in (1, 2, 4, 5, 8, 16, 19)}
    before = {b: m(x) for b, x in xs.items()}
    assert m.prepack()
    for b, x in xs.items():
        got = m(x)
        assert orc.rel_l2(got.float().cpu().numpy(), before[b].float().cpu().numpy().astype(np.float64)) <= 5e-4, b
        if b in (5, 19):
            assert torch.equal(got, before[b]), b   # same kernel as before
        assert torch.equal(got, m(x)), b
    m.prepack(release_reference=True)
    for b, x in xs.items():
        assert orc.rel_l2(m(x).float().cpu().numpy(), before[b].float().cpu().numpy().astype(np.float64)) <= 5e-4, b


def _column_sample(p, cols):
    return {"cherry_indices": p["cherry_indices"], "cherry_weight": np.ascontiguousarray(p["cherry_weight"][:, cols]),
            "qweight": np.ascontiguousarray(p["qweight"][:, cols]), "scales": np.ascontiguousarray(p["scales"][:, cols])}


@pytest.mark.parametrize("bits,k,n", [(4, 8192, 28672), (3, 8192, 28672), (3, 8192, 16392), (4, 8192, 16392),
                                      (4, 28672, 8192), (3, 28672, 8192)])
def test_prepacked_deep_and_wide_layers_walk_tiles(qc, bits, k, n):
    """64 units per column AND more tiles than resident workgroups: the geometry a loader selects for
    the 70B gate / up projections (computing wavefronts that stage the activations themselves, every
    workgroup walking several tiles).  C oracle on a column sample that covers the first and the
    last tile and tiles a workgroup takes second and last; one-hot columns bit for bit; accumulate;
    repeatable."""
    announce("prepacked deep+wide", bits, k, n)
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=41 + bits)
    c = p["cherry_indices"].shape[0]
    stream = prepack(qc, bits, p, k)
    rng = np.random.default_rng(13)
    x = rng.standard_normal((1, k)).astype(np.float16)
    y = run(qc, bits, stream, x, n, c)
    assert np.isfinite(y).all()
    ntiles = -(-n // 16)
    tiles = sorted(set([0, 1, 255, 256, 257, 511, 512, 767, 768, 1023, 1024, ntiles // 2, ntiles - 2, ntiles - 1])
                   | set(int(t) for t in rng.choice(ntiles, size=18, replace=False)))
    tiles = [t for t in tiles if t < ntiles]
    cols = np.array([c0 for t in tiles for c0 in range(16 * t, min(n, 16 * t + 16))])
    sub = _column_sample(p, cols)
    want = c_oracle.fused(x, sub, bits, 128)
    assert orc.rel_l2(y[:, cols], want) <= TOL
    ulp_ok = np.abs(y[:, cols].astype(np.float64) - want) <= np.abs(want) * 2 ** -10 + 1e-3
    assert ulp_ok.mean() > 0.999
    np.testing.assert_array_equal(run(qc, bits, stream, x, n, c), y)
    base = rng.standard_normal((1, n)).astype(np.float16)
    ya = run(qc, bits, stream, x, n, c, out=base.copy(), accumulate=True)
    assert orc.rel_l2(ya[:, cols], want + base[:, cols].astype(np.float64)) <= TOL
    # linearity over the whole width: every tile of every workgroup, not only the sample
    y2 = run(qc, bits, stream, (x * np.float16(2)).astype(np.float16), n, c)
    np.testing.assert_array_equal(y2, (y.astype(np.float32) * 2).astype(np.float16))
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    kn = len(nidx)
    for j in [int(nidx[0]), int(nidx[127]), int(nidx[128]), int(nidx[4095]), int(nidx[4096]), int(nidx[kn - 1]),
              int(nidx[kn - 129]), int(nidx[kn // 2 + 77]), int(idx[0]), int(idx[-1])]:
        e = np.zeros((1, k), dtype=np.float16)
        e[0, j] = 1
        with np.errstate(over="ignore"):
            np.testing.assert_array_equal(run(qc, bits, stream, e, n, c)[:, cols],
                                          c_oracle.fused(e, sub, bits, 128).astype(np.float16), err_msg=f"column {j}")


@pytest.mark.parametrize("bits", [4, 3])
@pytest.mark.parametrize("case", ["qkv_gqa_norm", "gate_up_norm", "qkv_gqa_plain", "gate_up_plain"])
def test_prepacked_group_llama70b_shapes_against_the_c_oracle(bits, case):
    """The grouped launch at the 70B decoder's shapes (8192 input channels = 64 units per column):
    q / k / v with grouped-query widths 8192 / 1024 / 1024 and gate / up 2 x 28672, with and without
    the fused RMSNorm.  C oracle on a column sample per member (all columns for the narrow ones),
    one-hot through the norm bit for bit."""
    import cherryq_decoder as dec
    print("[case] prepacked group 70B", bits, case, flush=True)
    K = 8192
    widths = (8192, 1024, 1024) if case.startswith("qkv") else (28672, 28672)
    gen = torch.Generator(device="cuda").manual_seed(29 + bits)
    cfg = dec.DecoderConfig(w_bits=bits, group_size=128, cherry_fraction=1 / 256)
    mods = [dec.random_packed_linear(cfg, K, n, gen, "cuda") for n in widths]
    packed = [{b: getattr(m, b).cpu().numpy() for b in NAMES} for m in mods]
    for m in mods:
        assert m.prepack()
    f16 = lambda a: np.asarray(a).astype(np.float16)
    rng = np.random.default_rng(17)
    samples = []
    for n in widths:
        nt = n // 16
        tiles = sorted(set([0, 1, nt // 2, nt - 2, nt - 1]) | set(int(t) for t in rng.choice(nt, size=min(nt, 27), replace=False)))
        samples.append(np.array([c0 for t in tiles for c0 in range(16 * t, 16 * t + 16)]))
    subs = [_column_sample(p, cols) for p, cols in zip(packed, samples)]

    def go(vec, **kw):
        outs = [torch.full((1, n), 7.0, dtype=torch.float16, device="cuda") for n in widths]
        dec.matvec_group_prepacked(mods, torch.from_numpy(vec).cuda(), outs, **kw)
        torch.cuda.synchronize()
        return [o.cpu().numpy() for o in outs]

    if case.endswith("norm"):
        eps = 1e-6
        h = f16(rng.standard_normal((1, K)) * 3)
        nw = f16(rng.random(K) + 0.5)
        hf = h.astype(np.float64)
        act = f16(nw.astype(np.float64) * f16(hf / np.sqrt(np.mean(hf * hf) + eps)).astype(np.float64))
        got = go(h, norm_weight=torch.from_numpy(nw).cuda(), eps=eps)
        for o, sub, cols in zip(got, subs, samples):
            assert np.isfinite(o).all()
            assert orc.rel_l2(o[:, cols], c_oracle.fused(act, sub, bits, 128)) <= 1e-3
        again = go(h, norm_weight=torch.from_numpy(nw).cuda(), eps=eps)
        for a, b in zip(got, again):
            np.testing.assert_array_equal(a, b)
        nw2 = f16(2.0 ** rng.integers(-2, 3, K))
        for j in (0, 127, 128, 4097, K - 1, int(packed[0]["cherry_indices"][0]), int(packed[-1]["cherry_indices"][-1])):
            x = np.zeros((1, K), dtype=np.float16)
            x[0, j] = 1
            got = go(x, norm_weight=torch.from_numpy(nw2).cuda(), eps=1.0 - 1.0 / K)
            xa = np.zeros((1, K), dtype=np.float16)
            xa[0, j] = nw2[j]
            for o, sub, cols in zip(got, subs, samples):
                with np.errstate(over="ignore"):
                    np.testing.assert_array_equal(o[0, cols], f16(c_oracle.fused(xa, sub, bits, 128)[0]), err_msg=f"column {j}")
    else:
        x = f16(rng.standard_normal((1, K)))
        got = go(x)
        for o, sub, cols in zip(got, subs, samples):
            assert np.isfinite(o).all()
            assert orc.rel_l2(o[:, cols], c_oracle.fused(x, sub, bits, 128)) <= 1e-3
        for j in (0, 129, K - 1, int(packed[0]["cherry_indices"][3])):
            e = np.zeros((1, K), dtype=np.float16)
            e[0, j] = 1
            got = go(e)
            for i, (o, sub, cols) in enumerate(zip(got, subs, samples)):
                with np.errstate(over="ignore"):
                    np.testing.assert_array_equal(o[:, cols], f16(c_oracle.fused(e, sub, bits, 128)), err_msg=f"column {j} member {i}")


@pytest.mark.parametrize("bits,k,n,b", [(4, 512, 4608, 1), (3, 512, 4608, 1), (4, 640, 264, 1), (4, 512, 264, 2), (3, 512, 264, 5),
                                        (4, 512, 1032, 16), (3, 640, 264, 2), (4, 640, 520, 5), (3, 640, 4112, 16),
                                        (4, 256, 264, 9), (3, 136, 32, 16), (4, 136, 4608, 1), (4, 896, 264, 16)])
def test_prepacked_layers_with_fewer_units_than_wavefronts(bits, k, n, b):
    """Columns of 1 to 7 units: fewer than the 8 wavefronts of a team, so most wavefronts have no unit
    at all and must contribute exactly zero, whatever the LDS behind the staged activations holds."""
    import quant_cuda
    print("[case] prepacked short columns", bits, k, n, b, flush=True)
    p = orc.synthetic_layer(k, n, bits, 128, seed=80 + bits, cherry_fraction=1 / 64)[1]  # 8 or 16 cherry channels
    t = {name: torch.from_numpy(np.ascontiguousarray(v)).cuda() for name, v in p.items() if name in NAMES}
    c = int(p["cherry_indices"].shape[0])
    assert quant_cuda.prepack_supported(bits, b, k, n, c, 128)
    stream = quant_cuda.prepack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"], t["scales"], k, 128)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((b, k)).astype(np.float16)
    # fill LDS-sized garbage first: a kernel that leaves NaN patterns in LDS for the next workgroup
    junk = torch.full((1 << 20,), float("nan"), dtype=torch.float16, device="cuda")
    (junk * 1).sum()

    def go(xv):
        out = torch.full((xv.shape[0], n), 5.0, dtype=torch.float16, device="cuda")
        quant_cuda.matvec_prepacked_cherryq(bits, torch.from_numpy(xv).cuda(), stream, out, k, c)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    want = c_oracle.fused(x, p, bits, 128)
    for rep in range(3):
        got = go(x)
        assert np.isfinite(got).all(), rep
        for r in range(b):
            assert orc.rel_l2(got[r], want[r]) <= 1e-3, (rep, r)
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    pool = [int(nidx[0]), int(nidx[31]), int(nidx[-1]), int(nidx[len(nidx) // 2])] + ([int(idx[0]), int(idx[-1])] if len(idx) else [])
    e = np.zeros((b, k), dtype=np.float16)
    for r in range(b):
        e[r, pool[r % len(pool)]] = np.float16(2.0 ** ((r * 5) % 13 - 6))
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(go(e), c_oracle.fused(e, p, bits, 128).astype(np.float16))


@pytest.mark.parametrize("bits,k,n", [(4, 11008, 4096), (3, 11008, 4096), (4, 4096, 1024), (3, 13824, 5120), (4, 28672, 1032)])
def test_prepacked_gated_down_projection(bits, k, n):
    """cherryq_decode_matvec_gated_prepacked_f16: fp16(fp16(silu(gate)) * up) formed while the row is
    staged, then the matvec over the repacked layer, accumulating or not.  Against the C oracle's
    fused product of that activation, against the checkpoint-layout launch with the same prologue, and
    bit for bit where the activation is one-hot (silu(g) * u exactly representable)."""
    import cherryq_decoder as dec
    print("[case] prepacked gated", bits, k, n, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(31 + bits)
    cfg = dec.DecoderConfig(w_bits=bits, group_size=128, cherry_fraction=1 / 256)
    m = dec.random_packed_linear(cfg, k, n, gen, "cuda")
    p = {b: getattr(m, b).cpu().numpy() for b in NAMES}
    assert m.prepack()
    rng = np.random.default_rng(19)
    f16 = lambda a: np.asarray(a).astype(np.float16)
    up = f16(rng.standard_normal((1, k)))
    gate = f16(rng.standard_normal((1, k)) * 2)

    def act_of(g, u):
        g32 = g.astype(np.float32)
        silu = f16(g32 / (np.float32(1) + np.exp(-g32, dtype=np.float32)))
        return f16(silu.astype(np.float32) * u.astype(np.float32))

    def go(u, g, base=None):
        out = torch.full((1, n), 3.0, dtype=torch.float16, device="cuda") if base is None else torch.from_numpy(base).cuda()
        dec.matvec_gated_prepacked(m, torch.from_numpy(u).cuda(), torch.from_numpy(g).cuda(), out, accumulate=base is not None)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    act = act_of(gate, up)
    want = c_oracle.fused(act, p, bits, 128)
    got = go(up, gate)
    assert np.isfinite(got).all()
    assert orc.rel_l2(got, want) <= 1e-3
    np.testing.assert_array_equal(got, go(up, gate))
    base = f16(rng.standard_normal((1, n)))
    assert orc.rel_l2(go(up, gate, base), want + base.astype(np.float64)) <= 1e-3
    # the checkpoint-layout launch with the same prologue: same activation bits, two summation orders
    ref = torch.zeros(1, n, dtype=torch.float16, device="cuda")
    dec.matvec_group([m], torch.from_numpy(up).cuda(), [ref], vec_gate=torch.from_numpy(gate).cuda())
    torch.cuda.synchronize()
    assert orc.rel_l2(got, ref.cpu().numpy().astype(np.float64)) <= 5e-4
    # one-hot activations: gate = 0 everywhere (silu(0) = 0) except one channel with a huge gate
    # (silu(g) = g exactly in fp16 for g >= 17: exp(-g) < 2^-24)
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    for j in (int(nidx[0]), int(nidx[129]), int(nidx[-1]), int(idx[0]), int(idx[-1]), int(nidx[len(nidx) // 2])):
        g = np.zeros((1, k), dtype=np.float16)
        g[0, j] = 32
        u = f16(rng.standard_normal((1, k)))
        u[0, j] = np.float16(2.0 ** -5)
        e = np.zeros((1, k), dtype=np.float16)
        e[0, j] = 1   # 32 * 2^-5
        with np.errstate(over="ignore"):
            np.testing.assert_array_equal(go(u, g), f16(c_oracle.fused(e, p, bits, 128)), err_msg=f"column {j}")


def test_prepacked_gated_rejections():
    import cherryq_decoder as dec
    lib = dec._lib
    fake = 1 << 12
    f = lib.cherryq_decode_matvec_gated_prepacked_f16
    assert f(5, fake, fake, fake, 1 << 30, fake, 4096, 4096, 16, 0, None) == -5
    assert f(4, fake, None, fake, 1 << 30, fake, 4096, 4096, 16, 0, None) == -1
    assert f(4, fake, fake + 2, fake, 1 << 30, fake, 4096, 4096, 16, 0, None) == -6
    assert f(4, fake, fake, fake, 64, fake, 4096, 4096, 16, 0, None) == -4
    assert f(4, fake, fake, fake, 1 << 30, fake, 65536, 4096, 0, 0, None) == -7


@pytest.mark.parametrize("bits,k,n,norm", [(4, 4096, 11008, True), (3, 4096, 11008, True), (4, 4096, 11008, False),
                                           (4, 8192, 28672, True), (3, 8192, 4104, False), (4, 4096, 32008, True),
                                           (3, 1024, 264, True), (4, 512, 40, False),
                                           # the 48-unit geometry (LLaMA-13B: 5120 -> 13824), both widths, walking and not
                                           (3, 5120, 13824, True), (4, 5120, 13824, False), (4, 6144, 4104, True),
                                           (3, 6144, 264, False), (3, 8192, 28672, True)])
def test_prepacked_gate_up_fused_activation(bits, k, n, norm):
    """cherryq_decode_gate_up_prepacked_f16: both projections and SiLU(gate) * up in one launch.  Bit for
    bit what the separate launches give (grouped gate / up launch, then the SiLU * up kernel: same
    rounding points), and the activation of the C oracle's two products within tolerance."""
    import cherryq_decoder as dec
    print("[case] prepacked gate/up fused", bits, k, n, norm, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(37 + bits)
    cfg = dec.DecoderConfig(w_bits=bits, group_size=128, cherry_fraction=1 / 256)
    mg, mu = dec.random_packed_linear(cfg, k, n, gen, "cuda"), dec.random_packed_linear(cfg, k, n, gen, "cuda")
    packed = [{b: getattr(m, b).cpu().numpy() for b in NAMES} for m in (mg, mu)]
    assert mg.prepack() and mu.prepack()
    assert dec.gate_up_prepacked_supported(mg, mu)
    rng = np.random.default_rng(23)
    f16 = lambda a: np.asarray(a).astype(np.float16)
    # activations scaled so that the gate results spread over a few units: SiLU in its curved range
    x = f16(rng.standard_normal((1, k)) * 4)
    nw = f16(rng.random(k) + 0.5)
    eps = 1e-6
    kw = dict(norm_weight=torch.from_numpy(nw).cuda(), eps=eps) if norm else {}
    xt = torch.from_numpy(x).cuda()
    act = torch.full((1, n), 9.0, dtype=torch.float16, device="cuda")
    dec.gate_up_prepacked(mg, mu, xt, act, **kw)
    torch.cuda.synchronize()
    got = act.cpu().numpy()
    assert np.isfinite(got).all()
    # the separate launches
    g = torch.empty(1, n, dtype=torch.float16, device="cuda")
    u = torch.empty(1, n, dtype=torch.float16, device="cuda")
    dec.matvec_group_prepacked([mg, mu], xt, [g, u], **kw)
    want = torch.empty(1, n, dtype=torch.float16, device="cuda")
    dec._ok(dec._lib.cherryq_decode_silu_mul_f16(g.data_ptr(), u.data_ptr(), want.data_ptr(), n, dec._stream()), "silu_mul")
    torch.cuda.synchronize()
    # both launches round the same fp32 sums once: the last bit of gate or up may differ where the summation
    # orders differ (teams of two wavefronts here, of four there), never more
    gw, ww = got.astype(np.float64), want.cpu().numpy().astype(np.float64)
    assert orc.rel_l2(gw, ww) <= 5e-4
    assert (got == want.cpu().numpy()).mean() > 0.8
    # against the oracle
    if norm:
        hf = x.astype(np.float64)
        a_in = f16(nw.astype(np.float64) * f16(hf / np.sqrt(np.mean(hf * hf) + eps)).astype(np.float64))
    else:
        a_in = x
    cols = np.arange(n) if k * n <= 4096 * 11008 else np.sort(rng.choice(n // 16, size=40, replace=False))[:, None] * 16 + np.arange(16)
    cols = np.asarray(cols).reshape(-1)
    subs = [_column_sample(p, cols) for p in packed]
    go, uo = (f16(c_oracle.fused(a_in, sp, bits, 128)) for sp in subs)
    g32 = go.astype(np.float32)
    silu = f16(g32 / (np.float32(1) + np.exp(-g32, dtype=np.float32)))
    ref = f16(silu.astype(np.float32) * uo.astype(np.float32)).astype(np.float64)
    assert orc.rel_l2(gw[:, cols], ref) <= 2e-3   # fp16 roundings of gate and up enter the activation
    # repeatable
    act2 = torch.empty_like(act)
    dec.gate_up_prepacked(mg, mu, xt, act2, **kw)
    torch.cuda.synchronize()
    assert torch.equal(act, act2)
