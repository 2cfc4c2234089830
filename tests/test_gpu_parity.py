"""Parity of the HIP path with the CPU oracle on identical packed inputs (MI355X only).

Bars: dequantised weights bit-exact; fused outputs within rel-L2 <= 1e-3 of the oracle's
dequantise-and-matmul (fp16 weights, wide accumulation, one rounding); one-hot activations read
dequantised weights back through the fused kernels bit for bit.
"""
import ctypes
import glob
import os
import sys

import numpy as np
import pytest
import torch

from oracle import cherryq_oracle as orc
from oracle import c_oracle

pytestmark = pytest.mark.gpu

TOL = 1e-3  # rel-L2 bar on fused outputs
GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "golden_*.npz")))
NAMES = ("cherry_indices", "cherry_weight", "qweight", "scales")


@pytest.fixture(scope="module")
def qc():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import quant_cuda
    return quant_cuda


def dev(packed):
    return {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in packed.items() if k in NAMES}


def announce(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def run_fused(qc, bits, x, p, gs, mul=None):
    d = dev(p)
    xt = torch.from_numpy(x).cuda()
    out = torch.zeros(x.shape[0], p["qweight"].shape[1], dtype=torch.float16, device="cuda") if mul is None \
        else torch.from_numpy(mul).cuda()
    if bits == 4:
        qc.vecquant4matmul_cherryq(xt, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], out, gs)
    else:
        qc.vecquant3matmul_cherryq(xt, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], out,
                                   gs, True)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def oracle_outputs(bits, x, p, gs):
    k = x.shape[1]
    dense = c_oracle.unpack(p, bits, gs, k)
    y_deq = c_oracle.linear(x, dense, want_f64=True)[1]   # fp16 weights, wide accumulation
    y_fused = c_oracle.fused(x, p, bits, gs)               # un-rounded weights, wide accumulation
    return dense, y_deq, y_fused


# ------------------------------------------------------------------------- golden fixtures

@pytest.mark.parametrize("path", [p for p in GOLDEN if "_f32" not in p and "gall" not in p],
                         ids=lambda p: os.path.basename(p)[7:-4])
def test_fused_on_golden_fixtures(qc, path):
    d = np.load(path)
    bits, gs, k, n, c = (int(v) for v in d["meta"])
    announce("golden", os.path.basename(path), bits, gs, k, n, c)
    if bits == 4 and gs < 128:
        pytest.skip("4-bit needs group_size >= 128, as in the reference")
    p = {name: d[name] for name in NAMES}
    y = run_fused(qc, bits, d["x"], p, gs)
    assert orc.rel_l2(y, d["forward_dequantized"]) <= 2 * TOL  # reference's own fp16 CPU linear
    _, y_deq, y_fused = oracle_outputs(bits, d["x"], p, gs)
    assert orc.rel_l2(y, y_deq) <= TOL
    assert orc.rel_l2(y, y_fused) <= TOL


@pytest.mark.parametrize("path", [p for p in GOLDEN if "_f32" not in p], ids=lambda p: os.path.basename(p)[7:-4])
def test_unpack_kernel_bit_exact_on_golden(qc, path):
    d = np.load(path)
    bits, gs, k, n, c = (int(v) for v in d["meta"])
    announce("unpack golden", os.path.basename(path))
    t = dev({name: d[name] for name in NAMES})
    g = gs if gs != -1 else k
    dense = qc.unpack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"], t["scales"], k, g)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(dense.cpu().numpy(), d["unpack"])


# ------------------------------------------------------------------------- full-size shapes

SHAPES_B1 = [
    (4, 4096, 4096), (3, 4096, 4096),            # config 0 (+ its 3-bit twin)
    (4, 4096, 11008), (3, 4096, 11008),          # config 1: gate / up
    (4, 11008, 4096), (3, 11008, 4096),          # config 1: down
    (3, 5120, 5120), (3, 5120, 13824), (3, 13824, 5120),   # config 3 (13B)
    (4, 8192, 1024), (4, 8192, 8192),            # config 4 (70B), smaller two
]


@pytest.mark.parametrize("bits,k,n", SHAPES_B1)
def test_matvec_baseline_shapes(qc, bits, k, n):
    announce("matvec", bits, k, n)
    w, p = orc.synthetic_layer(k, n, bits, 128, seed=k + n + bits)
    rng = np.random.default_rng(7)
    x = rng.standard_normal((1, k)).astype(np.float16)
    y = run_fused(qc, bits, x, p, 128)
    _, y_deq, y_fused = oracle_outputs(bits, x, p, 128)
    e_deq, e_fused = orc.rel_l2(y, y_deq), orc.rel_l2(y, y_fused)
    print(f"  rel-L2 vs dequant-matmul {e_deq:.2e}, vs un-rounded contract {e_fused:.2e}")
    assert e_deq <= TOL and e_fused <= TOL
    # the result is the fp16 rounding of the fp32 sum: compare against the rounded contract
    ulp_ok = np.abs(y.astype(np.float64) - y_fused) <= np.abs(y_fused) * 2 ** -10 + 1e-3
    assert ulp_ok.mean() > 0.999


@pytest.mark.parametrize("bits,k,n", [(4, 8192, 28672), (4, 28672, 8192)])
def test_matvec_70b_large_shapes_properties(qc, bits, k, n):
    """Full-size 70B shapes: random packed bytes (no quantisation pass), checked against the C
    oracle on a column sample and through linearity."""
    announce("matvec-large", bits, k, n)
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=3)
    rng = np.random.default_rng(11)
    x1 = rng.standard_normal((1, k)).astype(np.float16)
    y1 = run_fused(qc, bits, x1, p, 128)
    cols = np.sort(rng.choice(n, size=512, replace=False))
    sub = {"cherry_indices": p["cherry_indices"], "cherry_weight": np.ascontiguousarray(p["cherry_weight"][:, cols]),
           "qweight": np.ascontiguousarray(p["qweight"][:, cols]), "scales": np.ascontiguousarray(p["scales"][:, cols])}
    want = c_oracle.fused(x1, sub, bits, 128)
    assert orc.rel_l2(y1[:, cols], want) <= TOL
    # linearity: f(2 x) == 2 f(x) exactly (powers of two commute with every rounding involved)
    y2 = run_fused(qc, bits, (x1 * np.float16(2)).astype(np.float16), p, 128)
    np.testing.assert_array_equal(y2, (y1.astype(np.float32) * 2).astype(np.float16))


@pytest.mark.parametrize("bits,k,n", [(4, 4096, 4096), (3, 4096, 4096), (4, 11008, 512), (3, 11008, 512)])
def test_one_hot_reads_back_dequantised_weights(qc, bits, k, n):
    """x = e_j returns column j of the dense weight: the fused decode is bit-exact."""
    announce("one-hot", bits, k, n)
    w, p = orc.synthetic_layer(k, n, bits, 128, seed=5)
    dense = c_oracle.unpack(p, bits, 128, k)
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    probes = [int(nidx[0]), int(nidx[1]), int(nidx[127]), int(nidx[128]), int(nidx[-1]), int(nidx[-113]),
              int(idx[0]), int(idx[-1]), int(idx[0]) + 1 if idx[0] + 1 not in idx else int(nidx[5]),
              int(nidx[len(nidx) // 2 + 3])]
    for j in probes:
        x = np.zeros((1, k), dtype=np.float16)
        x[0, j] = 1
        y = run_fused(qc, bits, x, p, 128)
        np.testing.assert_array_equal(y[0], dense[:, j], err_msg=f"column {j}")
    # a single small activation: the output is the exact product (code - c_b) * scale * x rounded
    # once to fp16 (here into the subnormal range, where rounding the weight first would differ)
    x = np.zeros((1, k), dtype=np.float16)
    x[0, probes[2]] = np.float16(2 ** -9)
    y = run_fused(qc, bits, x, p, 128)
    np.testing.assert_array_equal(y[0], c_oracle.fused(x, p, bits, 128)[0].astype(np.float16))


def test_accumulate_semantics_and_repeat_calls(qc):
    """mul += result, like the reference entry point; repeated calls keep accumulating and the
    split-K counters come back to zero every time."""
    announce("accumulate")
    bits, k, n = 4, 4096, 4096
    w, p = orc.synthetic_layer(k, n, bits, 128, seed=2)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, k)).astype(np.float16)
    init = rng.standard_normal((1, n)).astype(np.float16)
    d = dev(p)
    xt = torch.from_numpy(x).cuda()
    mul = torch.from_numpy(init).cuda()
    y_fused = c_oracle.fused(x, p, bits, 128)
    expect = init.astype(np.float64)
    for rep in range(3):
        qc.vecquant4matmul_cherryq(xt, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], mul, 128)
        torch.cuda.synchronize()
        expect = (expect + y_fused).astype(np.float16).astype(np.float64)
        assert orc.rel_l2(mul.cpu().numpy(), expect) <= TOL, rep
    # determinism: same inputs, same bits
    a = run_fused(qc, bits, x, p, 128)
    b = run_fused(qc, bits, x, p, 128)
    np.testing.assert_array_equal(a, b)


def test_scale_invariance_small_and_large_activations(qc):
    announce("scale-invariance")
    for bits in (3, 4):
        k, n = 4096, 1024
        w, p = orc.synthetic_layer(k, n, bits, 128, seed=9)
        rng = np.random.default_rng(4)
        base = rng.standard_normal((1, k)).astype(np.float32)
        for scale in (2.0 ** -12, 2.0 ** -6, 1.0, 2.0 ** 6):
            x = (base * scale).astype(np.float16)
            y = run_fused(qc, bits, x, p, 128)
            assert orc.rel_l2(y, c_oracle.fused(x, p, bits, 128)) <= TOL, (bits, scale)


# ------------------------------------------------------------------------- batches / variants

@pytest.mark.parametrize("bits,k,n,b", [(3, 5120, 5120, 4), (3, 5120, 5120, 8), (3, 5120, 13824, 8),
                                        (4, 8192, 1024, 16), (4, 4096, 4096, 2), (4, 4096, 4096, 5),
                                        (3, 4096, 4096, 16), (4, 4096, 4096, 19)])
def test_small_batches(qc, bits, k, n, b):
    announce("batch", bits, k, n, b)
    w, p = orc.synthetic_layer(k, n, bits, 128, seed=b)
    rng = np.random.default_rng(b)
    x = rng.standard_normal((b, k)).astype(np.float16)
    y = run_fused(qc, bits, x, p, 128)
    _, y_deq, y_fused = oracle_outputs(bits, x, p, 128)
    assert orc.rel_l2(y, y_deq) <= TOL and orc.rel_l2(y, y_fused) <= TOL
    for r in range(b):
        assert orc.rel_l2(y[r], y_fused[r]) <= TOL, r


@pytest.mark.parametrize("bits,k,n", [(4, 4096, 4096), (3, 4096, 4096), (4, 11008, 512), (3, 5120, 768)])
def test_batch_one_hot_rows_are_bit_exact(qc, bits, k, n):
    """16 one-hot activation rows through the matrix-core path: row i returns dequantised column
    j_i bit for bit (subnormal code fields, per-row normalisation and the A/B operand order)."""
    announce("batch one-hot", bits, k, n)
    w, p = orc.synthetic_layer(k, n, bits, 128, seed=8)
    dense = c_oracle.unpack(p, bits, 128, k)
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    cols = [int(nidx[0]), int(nidx[1]), int(nidx[2]), int(nidx[3]), int(nidx[7]), int(nidx[8]), int(nidx[31]),
            int(nidx[32]), int(nidx[127]), int(nidx[128]), int(nidx[-1]), int(nidx[-9]), int(idx[0]), int(idx[7]),
            int(idx[8]), int(idx[-1])]
    x = np.zeros((16, k), dtype=np.float16)
    for i, j in enumerate(cols):
        x[i, j] = 1
    y = run_fused(qc, bits, x, p, 128)
    for i, j in enumerate(cols):
        np.testing.assert_array_equal(y[i], dense[:, j], err_msg=f"row {i} column {j}")
    # rows of very different magnitude in one batch; powers of two keep the products exact
    scale = np.array([2.0 ** e for e in (-14, -10, -6, -3, 0, 1, 3, 5, 7, 9, 11, 12, 13, 14, 15, 15)])
    xs = (x.astype(np.float64) * scale[:, None]).astype(np.float16)
    ys = run_fused(qc, bits, xs, p, 128)
    want = c_oracle.fused(xs, p, bits, 128)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(ys, want.astype(np.float16))


_ROWS_LAYERS = {}


@pytest.mark.parametrize("b", [2, 3, 4])
@pytest.mark.parametrize("bits,k,n", [(4, 4096, 4096), (3, 4096, 4096), (4, 4096, 11008), (3, 11008, 512)])
def test_two_to_four_one_hot_rows_are_bit_exact(qc, bits, k, n, b):
    """2, 3 and 4 one-hot activation rows (the two-row dot2 and the four-row 4x4x4 matrix-core
    instantiations of the streaming kernel): row i returns dequantised column j_i bit for bit, also
    with rows of very different power-of-two magnitude, for several placements of the columns."""
    announce("rows one-hot", bits, k, n, b)
    if (bits, k, n) not in _ROWS_LAYERS:  # the same layer serves the three row counts
        p = orc.synthetic_layer(k, n, bits, 128, seed=9)[1]
        _ROWS_LAYERS[(bits, k, n)] = (p, c_oracle.unpack(p, bits, 128, k))
    p, dense = _ROWS_LAYERS[(bits, k, n)]
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    pool = [int(nidx[0]), int(nidx[1]), int(nidx[63]), int(nidx[64]), int(nidx[127]), int(nidx[128]), int(nidx[-1]),
            int(nidx[-65]), int(idx[0]), int(idx[-1]), int(idx[len(idx) // 2]), int(nidx[len(nidx) // 2 + 5])]
    for start in range(0, len(pool), b):
        cols = [pool[(start + i) % len(pool)] for i in range(b)]
        x = np.zeros((b, k), dtype=np.float16)
        for i, j in enumerate(cols):
            x[i, j] = 1
        y = run_fused(qc, bits, x, p, 128)
        for i, j in enumerate(cols):
            np.testing.assert_array_equal(y[i], dense[:, j], err_msg=f"row {i} column {j}")
        # 2^-9 is the smallest factor that keeps every product (down to an fp16-subnormal cherry
        # weight, 2^-24) a multiple of the split-K accumulator's 2^-34 step
        scale = np.array([2.0 ** e for e in (-9, 3, -5, 9)][:b])
        xs = (x.astype(np.float64) * scale[:, None]).astype(np.float16)
        ys = run_fused(qc, bits, xs, p, 128)
        with np.errstate(over="ignore"):
            np.testing.assert_array_equal(ys, c_oracle.fused(xs, p, bits, 128).astype(np.float16))


@pytest.mark.parametrize("bits,k,n,b", [(4, 8192, 8192, 16), (4, 8192, 28672, 16), (4, 28672, 8192, 16),
                                        (3, 13824, 5120, 8), (3, 5120, 13824, 4)])
def test_batch_large_shapes(qc, bits, k, n, b):
    """Configs 3 and 4 at their batch sizes: random packed bytes, C oracle on a column sample."""
    announce("batch-large", bits, k, n, b)
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=4)
    rng = np.random.default_rng(b)
    x = rng.standard_normal((b, k)).astype(np.float16)
    y = run_fused(qc, bits, x, p, 128)
    cols = np.sort(rng.choice(n, size=256, replace=False))
    sub = {"cherry_indices": p["cherry_indices"], "cherry_weight": np.ascontiguousarray(p["cherry_weight"][:, cols]),
           "qweight": np.ascontiguousarray(p["qweight"][:, cols]), "scales": np.ascontiguousarray(p["scales"][:, cols])}
    assert orc.rel_l2(y[:, cols], c_oracle.fused(x, sub, bits, 128)) <= TOL
    # the batch path agrees with the batch-1 path row by row (different kernels, same contract)
    y0 = run_fused(qc, bits, x[:1], p, 128)
    assert orc.rel_l2(y[0], y0[0]) <= TOL


def test_batch_accumulate_scale_invariance_and_determinism(qc):
    announce("batch-misc")
    for bits in (3, 4):
        k, n, b = 4096, 1024, 8
        w, p = orc.synthetic_layer(k, n, bits, 128, seed=bits + 20)
        rng = np.random.default_rng(5)
        base = rng.standard_normal((b, k)).astype(np.float32)
        for scale in (2.0 ** -12, 2.0 ** -5, 1.0, 2.0 ** 5):
            x = (base * scale).astype(np.float16)
            y = run_fused(qc, bits, x, p, 128)
            assert orc.rel_l2(y, c_oracle.fused(x, p, bits, 128)) <= TOL, (bits, scale)
        x = base.astype(np.float16)
        init = rng.standard_normal((b, n)).astype(np.float16)
        y1 = run_fused(qc, bits, x, p, 128, mul=init.copy())
        want = (init.astype(np.float64) + c_oracle.fused(x, p, bits, 128))
        assert orc.rel_l2(y1, want) <= TOL
        np.testing.assert_array_equal(run_fused(qc, bits, x, p, 128), run_fused(qc, bits, x, p, 128))
        # the generic kernel (independent code) agrees
        qc.force_generic(True)
        try:
            yg = run_fused(qc, bits, x, p, 128)
        finally:
            qc.force_generic(False)
        assert orc.rel_l2(run_fused(qc, bits, x, p, 128), yg) <= TOL


@pytest.mark.parametrize("bits,gs,k,n,frac,b", [
    (3, 64, 1024, 512, 1 / 64, 1), (3, 64, 1024, 512, 1 / 64, 3),     # group 64 (reference G64 kernels)
    (4, 256, 2048, 512, 1 / 256, 1), (3, 256, 2048, 264, 1 / 256, 2),  # group 256, N not a multiple of 256
    (4, 128, 1024, 8, 1 / 256, 1),                                    # no cherries (K < 2048), tiny N
    (4, 128, 4096, 72, 1 / 16, 1), (3, 128, 4096, 72, 1 / 16, 4),     # 256 cherries: beyond the fast path
    (3, 32, 512, 256, 1 / 32, 1), (4, 4096, 4096, 256, 1 / 256, 1),   # group 32; one group for all of K
    (4, 128, 2048 + 8, 256, 1 / 256, 1), (3, 128, 2048 + 8, 256, 1 / 256, 1),  # ragged last unit (8 positions)
    (4, 128, 2048 + 8, 256, 1 / 256, 2), (3, 128, 2048 + 8, 264, 1 / 256, 4),  # the same with 2 and 4 rows in one pass
    (4, 128, 1024, 8, 1 / 256, 3), (3, 128, 4096, 1000, 1 / 32, 2),           # rows: tiny N; 128 cherries
])
def test_layout_variants(qc, bits, gs, k, n, frac, b):
    announce("variant", bits, gs, k, n, frac, b)
    w, p = orc.synthetic_layer(k, n, bits, gs, seed=13, cherry_fraction=frac)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((b, k)).astype(np.float16)
    y = run_fused(qc, bits, x, p, gs)
    _, y_deq, y_fused = oracle_outputs(bits, x, p, gs)
    assert orc.rel_l2(y, y_deq) <= TOL and orc.rel_l2(y, y_fused) <= TOL


def test_cherry_positions_edge_cases(qc):
    """Cherries at the very start / end, adjacent runs, and clustered inside one unit."""
    announce("cherry-edges")
    k, n, gs = 4096, 256, 128
    rng = np.random.default_rng(3)
    for bits in (3, 4):
        for idx in ([0, 1, 2, 3, 4, 5, 6, 7, 4088, 4089, 4090, 4091, 4092, 4093, 4094, 4095],
                    list(range(300, 316)),
                    [5, 127, 128, 129, 255, 256, 1000, 1001, 2047, 2048, 2049, 3000, 3071, 3072, 4000, 4095]):
            w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
            p = orc.pack(w, np.array(idx), bits, gs)
            x = rng.standard_normal((1, k)).astype(np.float16)
            y = run_fused(qc, bits, x, p, gs)
            assert orc.rel_l2(y, c_oracle.fused(x, p, bits, gs)) <= TOL, (bits, idx[:3])
            # every cherry column and its neighbours, one-hot
            dense = c_oracle.unpack(p, bits, gs, k)
            for j in sorted(set(idx[:3] + idx[-3:] + [min(idx[-1] + 1, k - 1), max(idx[0] - 1, 0)])):
                e = np.zeros((1, k), dtype=np.float16)
                e[0, j] = 1
                np.testing.assert_array_equal(run_fused(qc, bits, e, p, gs)[0], dense[:, j])


def test_fp32_entry_point_benchmark_speed_shape(qc):
    """vecquant3matmul_cherryq(..., fp16=False): fp32 tensors, int32 indices, batch 16, repeated
    accumulation into the same `mul` -- the call pattern of the reference's benchmark_speed.py."""
    announce("fp32")
    b, k, n, c = 16, 4096, 13824 // 8, 16
    rng = np.random.default_rng(0)
    vec = rng.standard_normal((b, k)).astype(np.float32)
    qweight = rng.integers(1, 5, size=(1530, n), dtype=np.uint8)
    cw = rng.standard_normal((c, n)).astype(np.float32)
    idx = np.arange(16, dtype=np.int32)
    scales = np.ones((32, n), dtype=np.float32)
    mul = torch.zeros(b, n, device="cuda")
    args = [torch.from_numpy(a).cuda() for a in (vec, qweight, cw, idx, scales)]
    for _ in range(2):
        qc.vecquant3matmul_cherryq(*args, mul, 128, False)
    torch.cuda.synchronize()
    u = orc.unpack_codes(qweight, 3).astype(np.float64) - 3.5
    nidx = orc.normal_indices(k, idx)
    want = 2 * (vec[:, nidx].astype(np.float64) @ u + vec[:, idx].astype(np.float64) @ cw.astype(np.float64))
    np.testing.assert_allclose(mul.cpu().numpy(), want, rtol=2e-5, atol=2e-3)


F32_CASES = [
    # b, k, n, cherries, group
    (16, 4096, 1728, 16, 128),     # the benchmark_speed.py call shape (columns / 8)
    (2, 1024, 256, 8, 128), (5, 1024, 264, 0, 128),        # N % 16 == 8, no cherries
    (16, 2048 + 40, 520, 40, 128),                          # ragged last unit, two cherry units, N % 256 != 0
    (17, 1024, 512, 8, 256), (40, 2048, 256, 32, 1024),     # more than one pass of 16 rows; wide groups
    (3, 1024, 256, 8, 64), (1, 1024, 256, 8, 128),          # group 64: generic kernel; one row: matrix-core kernel
]


@pytest.mark.parametrize("b,k,n,c,g", F32_CASES, ids=[f"b{v[0]}-k{v[1]}-n{v[2]}-c{v[3]}-g{v[4]}" for v in F32_CASES])
def test_fp32_variant_against_float64(qc, b, k, n, c, g):
    """fp32 tensors, int32 indices: the matrix-core kernel (2 rows and more, groups of whole units)
    and the generic kernel against a float64 evaluation, and against each other."""
    announce("fp32 variant", b, k, n, c, g)
    rng = np.random.default_rng(1000 * b + k + n + c)
    kn = k - c
    vec = rng.standard_normal((b, k)).astype(np.float32)
    qweight = rng.integers(0, 256, size=(kn // 8 * 3, n), dtype=np.uint8)
    cw = rng.standard_normal((c, n)).astype(np.float32)
    idx = np.sort(rng.choice(k, c, replace=False)).astype(np.int32)
    scales = (rng.random((-(-kn // g), n)) * 0.01 + 0.005).astype(np.float32)
    init = rng.standard_normal((b, n)).astype(np.float32)
    u = orc.unpack_codes(qweight, 3).astype(np.float64) - 3.5
    wn = u * np.repeat(scales.astype(np.float64), g, axis=0)[:kn]
    nidx = orc.normal_indices(k, idx)
    want = init + vec[:, nidx].astype(np.float64) @ wn + vec[:, idx].astype(np.float64) @ cw.astype(np.float64)
    args = [torch.from_numpy(a).cuda() for a in (vec, qweight, cw, idx, scales)]

    def run():
        mul = torch.from_numpy(init.copy()).cuda()
        qc.vecquant3matmul_cherryq(*args, mul, g, False)
        torch.cuda.synchronize()
        return mul.cpu().numpy()

    got = run()
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-6 * scale * np.sqrt(k / 1024)
    np.testing.assert_array_equal(got, run())           # order-independent accumulation
    qc.force_generic(True)
    try:
        generic = run()
    finally:
        qc.force_generic(False)
    assert np.abs(generic - want).max() <= 2e-6 * scale * np.sqrt(k / 1024)


def test_fp32_variant_single_row_with_and_without_scratch_through_the_c_abi(qc):
    """One fp32 row: without a scratch buffer the call takes the generic kernel, with
    cherryq_scratch_bytes_f32() bytes the matrix-core kernel; both leave the workspace zeroed."""
    announce("fp32 c-abi one row")
    lib = qc._lib
    k, n, c, g = 2048, 512, 8, 128
    rng = np.random.default_rng(21)
    kn = k - c
    vec = rng.standard_normal((1, k)).astype(np.float32)
    qweight = rng.integers(0, 256, size=(kn // 8 * 3, n), dtype=np.uint8)
    cw = rng.standard_normal((c, n)).astype(np.float32)
    idx = np.sort(rng.choice(k, c, replace=False)).astype(np.int32)
    scales = (rng.random((-(-kn // g), n)) * 0.01 + 0.005).astype(np.float32)
    u = orc.unpack_codes(qweight, 3).astype(np.float64) - 3.5
    want = vec[:, orc.normal_indices(k, idx)].astype(np.float64) @ (u * np.repeat(scales.astype(np.float64), g, axis=0)[:kn]) \
        + vec[:, idx].astype(np.float64) @ cw.astype(np.float64)
    t = [torch.from_numpy(a).cuda() for a in (vec, qweight, cw, idx, scales)]
    ws_b = lib.cherryq_workspace_bytes(1, k, n, c)
    sc_b = lib.cherryq_scratch_bytes_f32(1, k, n, c)
    assert lib.cherryq_scratch_bytes(1, k, n, c) == 0 and sc_b > 0
    ws = torch.zeros(ws_b, dtype=torch.uint8, device="cuda")
    sc = torch.empty(sc_b, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    lib.cherryq_vecquant3matmul_f32.argtypes = [ctypes.c_void_p] * 6 + [ctypes.c_int] * 6 + \
        [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    for scratch, nbytes in ((None, 0), (sc.data_ptr(), sc_b)):
        out = torch.zeros(1, n, device="cuda")
        rc = lib.cherryq_vecquant3matmul_f32(*(a.data_ptr() for a in t), out.data_ptr(), 1, k, n, c, g, 1,
                                             ws.data_ptr(), ws_b, scratch, nbytes, stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert np.abs(out.cpu().numpy() - want).max() <= 3e-6 * np.abs(want).max()
        assert not ws.any()


def test_fp32_variant_one_hot_rows_read_the_weights_back(qc):
    """One-hot activations through the fp32 matrix-core kernel return (code - 3.5) * scale and the
    cherry rows: every product is exact and every sum has one non-zero term, so the only
    deviation left is the split-K accumulator's fixed-point step of 2^-34."""
    announce("fp32 one-hot")
    k, n, c, g = 1024, 512, 8, 128
    rng = np.random.default_rng(7)
    kn = k - c
    qweight = rng.integers(0, 256, size=(kn // 8 * 3, n), dtype=np.uint8)
    cw = rng.standard_normal((c, n)).astype(np.float32)
    idx = np.sort(rng.choice(k, c, replace=False)).astype(np.int32)
    scales = (rng.random((kn // g + (kn % g > 0), n)) * 0.01 + 0.005).astype(np.float32)
    dense = np.zeros((k, n), np.float32)
    u = orc.unpack_codes(qweight, 3).astype(np.float32) - np.float32(3.5)
    dense[orc.normal_indices(k, idx)] = u * np.repeat(scales, g, axis=0)[:kn]
    dense[idx] = cw
    args = [torch.from_numpy(a).cuda() for a in (qweight, cw, idx, scales)]
    cols = np.concatenate([rng.choice(k, 13, replace=False), idx[:3]])
    x = np.zeros((16, k), np.float32)
    x[np.arange(16), cols] = 1.0
    mul = torch.zeros(16, n, device="cuda")
    qc.vecquant3matmul_cherryq(torch.from_numpy(x).cuda(), *args, mul, g, False)
    torch.cuda.synchronize()
    assert np.abs(mul.cpu().numpy().astype(np.float64) - dense[cols]).max() <= 2.0 ** -34


def test_unsupported_requests_raise(qc):
    announce("errors")
    k, n = 1024, 256
    w, p = orc.synthetic_layer(k, n, 4, 128, seed=1)
    d = dev(p)
    x = torch.zeros(1, k, dtype=torch.float16, device="cuda")
    out = torch.zeros(1, n, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 128"):
        qc.vecquant4matmul_cherryq(x, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], out, 64)
    with pytest.raises(RuntimeError):
        qc.vecquant4matmul_cherryq(x, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], out, 256)
    with pytest.raises(RuntimeError, match="contiguous"):
        qc.vecquant4matmul_cherryq(x, d["qweight"].t().contiguous().t(), d["cherry_weight"], d["cherry_indices"],
                                   d["scales"], out, 128)
    with pytest.raises(RuntimeError, match="dtype"):
        qc.vecquant4matmul_cherryq(x.float(), d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"],
                                   out, 128)
    with pytest.raises(RuntimeError):
        qc.vecquant4matmul_cherryq(x[:, :512].contiguous(), d["qweight"], d["cherry_weight"], d["cherry_indices"],
                                   d["scales"], out, 128)


# ------------------------------------------------------------------------- dense dequant

@pytest.mark.parametrize("bits,k,n,gs", [(4, 4096, 4096, 128), (3, 4096, 4096, 128), (3, 11008, 520, 128),
                                         (4, 2048, 264, 256), (3, 1024, 512, 64)])
def test_unpack_kernel_bit_exact(qc, bits, k, n, gs):
    announce("unpack", bits, k, n, gs)
    w, p = orc.synthetic_layer(k, n, bits, gs, seed=k)
    t = dev(p)
    dense = qc.unpack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"], t["scales"], k, gs)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(dense.cpu().numpy(), c_oracle.unpack(p, bits, gs, k))


@pytest.mark.parametrize("bits,k,n,frac", [(4, 8192, 28672, 1 / 256), (3, 8200, 16392, 1 / 32)])
def test_unpack_kernel_bit_exact_large(qc, bits, k, n, frac):
    """Launches big enough for a workgroup to walk several blocks of rows (the last one ragged),
    random codes, checked in slices of rows so that the host side stays small."""
    announce("unpack large", bits, k, n)
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=n, cherry_fraction=frac)
    t = dev(p)
    dense = qc.unpack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"], t["scales"], k, 128)
    torch.cuda.synchronize()
    for n0 in list(range(0, n, 4096)):
        n1 = min(n0 + 4096, n)
        part = {"cherry_indices": p["cherry_indices"], "cherry_weight": np.ascontiguousarray(p["cherry_weight"][:, n0:n1]),
                "qweight": np.ascontiguousarray(p["qweight"][:, n0:n1]), "scales": np.ascontiguousarray(p["scales"][:, n0:n1])}
        np.testing.assert_array_equal(dense[n0:n1].cpu().numpy(), c_oracle.unpack(part, bits, 128, k))


@pytest.mark.parametrize("bits,k,n,gs", [(3, 4096, 1024, 128), (4, 4096, 1024, 128), (4, 11008, 264, 128)])
def test_dequantize_normal_entry_points(qc, bits, k, n, gs):
    announce("DequantizeNormal", bits, k, n)
    w, p = orc.synthetic_layer(k, n, bits, gs, seed=k + 1)
    c = p["cherry_indices"].shape[0]
    s32 = p["scales"].astype(np.float32)
    out = torch.full((k, n), -1.0, device="cuda")
    fn = qc.Dequantize3Normal if bits == 3 else qc.Dequantize4Normal
    fn(torch.from_numpy(p["qweight"]).cuda(), torch.from_numpy(s32).cuda(), out, k, c, gs)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    np.testing.assert_array_equal(got[:k - c], c_oracle.dequantize_normal(p["qweight"], s32, bits, k, c, gs))
    assert np.all(got[k - c:] == -1.0)  # rows past Kn stay untouched


# ------------------------------------------------------------------------- module level

@pytest.mark.parametrize("bits", [3, 4])
def test_quantlinear_module_end_to_end(qc, bits):
    """pack() on the host, move to the GPU, fused forward vs dequantised forward vs oracle."""
    announce("module", bits)
    from llama.cherry_linear import QuantLinear as TrainLinear
    from llama.qlinear import QuantLinear as PackedLinear
    k, n = 4096, 512
    torch.manual_seed(bits)
    lin = TrainLinear(k, n, bias=True, w_bits=bits, group_size=128, cherryq=True).half()
    lin.weight.data.normal_(0, 0.02)
    lin.bias.data.normal_(0, 0.1)
    lin.eval()
    score = lin.weight.float().abs().amax(0)
    lin.register_cherry_indices(torch.argsort(score, descending=True)[:lin.num_cherries])
    q = PackedLinear(bits, 128, lin.quantizer, 1 / 256, k, n, bias=True)
    q.pack(lin)
    p = {name: getattr(q, name).numpy().copy() for name in NAMES}
    want_p = orc.pack(lin.weight.detach().numpy(), lin.cherry_indices.numpy(), bits, 128)
    for name in NAMES:
        np.testing.assert_array_equal(p[name], want_p[name], err_msg=name)
    q = q.cuda()
    x = torch.randn(2, 3, k, dtype=torch.float16, device="cuda")
    y = q(x)
    assert y.shape == (2, 3, n) and y.dtype == torch.float16
    xn = x.reshape(-1, k).cpu().numpy()
    want = c_oracle.fused(xn, p, bits, 128).astype(np.float16).astype(np.float64) + q.bias.cpu().numpy().astype(np.float64)
    assert orc.rel_l2(y.reshape(-1, n).cpu().numpy(), want) <= TOL
    dense_dev = q.unpack()
    np.testing.assert_array_equal(dense_dev.cpu().numpy(), c_oracle.unpack(p, bits, 128, k))
    with PackedLinear.dmode(layerwise_dequantize=False):
        y2 = q(x)
    assert q.dequantized
    assert orc.rel_l2(y2.reshape(-1, n).cpu().numpy(), want) <= 2 * TOL
    with pytest.raises(RuntimeError):
        q(x)  # fused mode after the packed buffers were dropped


def test_direct_c_abi_call_with_raw_pointers(qc):
    """The entry point as a non-Python host would call it: raw device pointers, explicit
    workspace, explicit stream."""
    announce("raw C ABI")
    bits, k, n = 4, 4096, 2048
    w, p = orc.synthetic_layer(k, n, bits, 128, seed=17)
    d = dev(p)
    c = p["cherry_indices"].shape[0]
    x = torch.randn(1, k, dtype=torch.float16, device="cuda")
    out = torch.full((1, n), 7.0, dtype=torch.float16, device="cuda")
    lib = ctypes.CDLL(qc.LIBRARY_PATH)
    lib.cherryq_workspace_bytes.restype = ctypes.c_size_t
    need = lib.cherryq_workspace_bytes(1, k, n, c)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.Stream()
    fn = lib.cherryq_vecquant4matmul_f16
    fn.argtypes = [ctypes.c_void_p] * 6 + [ctypes.c_int] * 6 + [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                                               ctypes.c_size_t, ctypes.c_void_p]
    fn.restype = ctypes.c_int
    torch.cuda.synchronize()
    rc = fn(x.data_ptr(), d["qweight"].data_ptr(), d["cherry_weight"].data_ptr(), d["cherry_indices"].data_ptr(),
            d["scales"].data_ptr(), out.data_ptr(), 1, k, n, c, 128, 0, ws.data_ptr(), need, None, 0,
            stream.cuda_stream)
    assert rc == 0
    stream.synchronize()
    want = c_oracle.fused(x.cpu().numpy(), p, bits, 128)
    assert orc.rel_l2(out.cpu().numpy(), want) <= TOL  # accumulate=0 overwrote the 7.0 fill
    assert int(ws.cpu().sum()) == 0  # every accumulator word is back to zero


# ------------------------------------------------------------------------- device-side pack
@pytest.mark.parametrize("bits", [3, 4])
def test_device_pack_is_bit_identical_to_host_pack(bits):
    """cherryq_pack_f16 against QuantLinear.pack() on the host (which the golden fixtures pin to
    the reference): every packed buffer equal byte for byte, on shapes with short last groups,
    groups that are not multiples of 128, ties, tiny and zero weights."""
    print("[case] device pack", bits, flush=True)
    import quant_cuda
    from llama.cherry_linear import QuantLinear as TrainLinear
    from llama.qlinear import QuantLinear
    gen = torch.Generator().manual_seed(11)
    for k, n, g, frac in ((256, 64, 128, 1 / 16), (1024, 328, 128, 1 / 64), (4096, 512, 128, 1 / 256),
                          (512, 136, 64, 1 / 32), (768, 72, 256, 1 / 32), (11008, 256, 128, 1 / 256)):
        lin = TrainLinear(k, n, bias=False, w_bits=bits, group_size=g, cherryq=True, cherry_fraction=frac).half()
        w = torch.randn(n, k, generator=gen) * 0.02
        w[torch.rand(n, k, generator=gen) < 0.01] *= 10
        w[0, :] = 0                                   # an all-zero row: scale from the 1e-6 floor alone
        w[1, : k // 2] = 1e-7                         # below fp16 resolution
        w = w.half()
        w[2] = (torch.randint(-8, 8, (k,), generator=gen).half() * 0.25)  # exact grid points: rounding ties
        with torch.no_grad():
            lin.weight.copy_(w)
        lin.register_cherry_indices(torch.randperm(k, generator=gen)[:lin.num_cherries])
        host = QuantLinear(bits, g, lin.quantizer, frac, k, n, bias=False)
        host.pack(lin)
        dev = QuantLinear(bits, g, lin.quantizer, frac, k, n, bias=False)
        dev.pack(lin.cuda())
        assert dev.qweight.is_cuda
        for name in ("cherry_indices", "cherry_weight", "scales", "qweight"):
            a, b = getattr(host, name), getattr(dev, name).cpu()
            assert a.dtype == b.dtype and a.shape == b.shape, (name, k, n, g)
            assert torch.equal(a, b), (name, k, n, g, int((a != b).sum()))
    with pytest.raises(RuntimeError):
        quant_cuda.pack_cherryq(bits, torch.zeros(8, 64, dtype=torch.float16, device="cuda"),
                                torch.tensor([1, 1, 2, 3, 4, 5, 6, 7]), 64)


# ------------------------------------------------------------------------- prompt-sized batches
def column_sample(p, rng, count):
    n = p["qweight"].shape[1]
    cols = np.sort(rng.choice(n, size=min(count, n), replace=False))
    sub = {"cherry_indices": p["cherry_indices"], "cherry_weight": np.ascontiguousarray(p["cherry_weight"][:, cols]),
           "qweight": np.ascontiguousarray(p["qweight"][:, cols]), "scales": np.ascontiguousarray(p["scales"][:, cols])}
    return cols, sub


@pytest.mark.parametrize("bits,gs,k,n,rows", [
    (4, 128, 4096, 1024, 17),      # one row tile, 8 K splits
    (3, 128, 4096, 1024, 128),
    (4, 128, 11008, 520, 96),      # N % 128 != 0, Kn % 64 != 0
    (3, 128, 1160, 264, 33),       # short K: few steps, ragged everything
    (3, 64, 2048, 256, 40),        # 3-bit with 64-wide groups
    (4, 256, 4096, 512, 70),       # groups of two steps... of four steps
    (4, 128, 28672, 512, 20),      # 112 cherry rows: two cherry steps
    (4, 128, 2048, 4096, 1100),    # nine row tiles, no K split
    (3, 128, 4096, 11008, 200),    # 7B gate/up, two row tiles
    (4, 128, 4096, 11008, 64),     # 64-row tiles: the whole call is one row tile
    (4, 128, 4096, 11008, 32),     # 32-row tiles: four wavefronts side by side, nine K splits
    (3, 64, 2048, 264, 24),        # 32-row tiles, 3-bit, 64-wide groups, ragged N
    (3, 128, 4096, 4096, 33),      # 64-row tiles, 3-bit
    (4, 128, 512, 98312, 40),      # 64-row tiles, more column tiles than resident workgroups: no K split
    (4, 128, 11008, 4096, 65),     # first row count on 128-row tiles again
])
def test_gemm_rows_against_oracle(qc, bits, gs, k, n, rows):
    """More than 16 rows: the tiled dequantise + MFMA kernel against the C oracle (a column sample
    for the large shapes), every row on its own as well."""
    announce("gemm", bits, gs, k, n, rows)
    p = orc.synthetic_packed_fast(k, n, bits, gs, seed=rows)
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, k)).astype(np.float16)
    y = run_fused(qc, bits, x, p, gs)
    cols, sub = column_sample(p, rng, 256)
    want = c_oracle.fused(x, sub, bits, gs)
    assert orc.rel_l2(y[:, cols], want) <= TOL
    for r in (0, 1, 15, 16, rows // 2, rows - 1):
        assert orc.rel_l2(y[r, cols], want[r]) <= TOL, r
    # against the dense path on the dequantised weight (fp16 weights, as this kernel uses them)
    dense = c_oracle.unpack(sub, bits, gs, k)
    assert orc.rel_l2(y[:, cols], c_oracle.linear(x, dense, want_f64=True)[1]) <= TOL


@pytest.mark.parametrize("bits,k,n", [(4, 4096, 1024), (3, 4096, 1024), (4, 11008, 520), (3, 1160, 264)])
def test_gemm_one_hot_rows_are_bit_exact(qc, bits, k, n):
    """One-hot activation rows through the tiled kernel: row i returns the dequantised weight
    column j_i bit for bit (field extraction, the exact u - c_b, the single rounding of the scale
    product, the position order shared by the A and B operands, the cherry steps)."""
    announce("gemm one-hot", bits, k, n)
    w, p = orc.synthetic_layer(k, n, bits, 128, seed=9)
    dense = c_oracle.unpack(p, bits, 128, k)
    idx = p["cherry_indices"].astype(np.int64)
    nidx = orc.normal_indices(k, idx)
    picks = [0, 1, 2, 3, 4, 5, 6, 7, 8, 31, 32, 63, 64, 65, 127, 128, len(nidx) - 1, len(nidx) - 2, len(nidx) - 9,
             len(nidx) // 2]
    cols = [int(nidx[i]) for i in picks] + [int(i) for i in idx]
    rng = np.random.default_rng(1)
    cols += [int(c) for c in rng.choice(k, size=150 - len(cols), replace=False)]   # spans two row tiles
    x = np.zeros((len(cols), k), dtype=np.float16)
    x[np.arange(len(cols)), cols] = 1
    y = run_fused(qc, bits, x, p, 128)
    np.testing.assert_array_equal(y, dense[:, cols].T)


def test_gemm_accumulate_linearity_and_determinism(qc):
    announce("gemm accumulate")
    bits, k, n, rows = 4, 4096, 2048, 150
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=2)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((rows, k)).astype(np.float16)
    y1 = run_fused(qc, bits, x, p, 128)
    y1b = run_fused(qc, bits, x, p, 128)
    np.testing.assert_array_equal(y1, y1b)                    # split-K partials are added in split order
    base = rng.standard_normal((rows, n)).astype(np.float16)
    y2 = run_fused(qc, bits, x, p, 128, mul=base.copy())     # the reference's accumulate-in-place contract
    cols, sub = column_sample(p, rng, 256)
    want = c_oracle.fused(x, sub, bits, 128)
    assert orc.rel_l2(y2[:, cols], want + base[:, cols].astype(np.float64)) <= TOL
    # f(2 x) == 2 f(x) exactly: powers of two commute with every rounding involved, except where
    # f(x) is an fp16 subnormal (its last bit is lost before the doubling)
    y4 = run_fused(qc, bits, (x * np.float16(2)).astype(np.float16), p, 128)
    normal = np.abs(y1.astype(np.float32)) >= 2.0 ** -14
    np.testing.assert_array_equal(y4[normal], (y1.astype(np.float32) * 2).astype(np.float16)[normal])
    assert np.abs(y4.astype(np.float32) - 2 * y1.astype(np.float32))[~normal].max(initial=0.0) <= 2.0 ** -23
    # rows do not interact: a row gives the same bits alone in a 17-row call padded with zeros
    x17 = np.zeros((17, k), dtype=np.float16)
    x17[3] = x[77]
    y17 = run_fused(qc, bits, x17, p, 128)
    assert not y17[[i for i in range(17) if i != 3]].any()
    assert orc.rel_l2(y17[3], y1[77].astype(np.float64)) <= 1e-3   # different split count: same contract


@pytest.mark.parametrize("bits,k,n,rows", [(4, 4096, 1024, 64), (3, 4096, 1024, 128), (4, 11008, 520, 96)])
def test_prefill_rows_dequantise_once_then_gemm(qc, bits, k, n, rows):
    """QuantLinear.forward at and above prefill_rows (dense library GEMM on the bit-exact dequantised
    weight) against the oracle's dequantised product, and against the fused kernel below the
    threshold."""
    announce("prefill", bits, k, n, rows)
    from llama.qlinear import QuantLinear as PackedLinear
    from llama.quantizer import FullSymQuantizer
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=rows)
    q = PackedLinear(bits, 128, FullSymQuantizer, 1 / 256, k, n, bias=False)
    for name in NAMES:
        setattr(q, name, torch.from_numpy(p[name]).cuda())
    x = np.random.default_rng(rows).standard_normal((rows, k)).astype(np.float16)
    saved = PackedLinear.prefill_rows
    try:
        PackedLinear.prefill_rows = 32
        y = q(torch.from_numpy(x).cuda())
        PackedLinear.prefill_rows = 1 << 30
        y_fused = q(torch.from_numpy(x).cuda())
    finally:
        PackedLinear.prefill_rows = saved
    assert y.shape == (rows, n) and y.dtype == torch.float16
    dense, y_deq, _ = oracle_outputs(bits, x, p, 128)
    assert orc.rel_l2(y.cpu().numpy(), y_deq) <= TOL
    assert orc.rel_l2(y_fused.cpu().numpy(), y_deq) <= TOL
    assert orc.rel_l2(y.cpu().numpy(), y_fused.cpu().numpy().astype(np.float64)) <= 2 * TOL


def test_gemm_buffers_are_checked_through_the_c_abi(qc):
    """Raw C-ABI call with 64 rows: buffers sized for 16 rows are refused (nothing is launched), the
    sizes the library asks for are accepted."""
    announce("gemm c-abi buffers")
    lib = qc._lib
    bits, k, n, rows = 4, 2048, 512, 64
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=5)
    d = dev(p)
    c = d["cherry_indices"].numel()
    x = torch.randn(rows, k, device="cuda").half()
    out = torch.full((rows, n), 5.0, dtype=torch.float16, device="cuda")
    small_ws, small_sc = lib.cherryq_workspace_bytes(16, k, n, c), lib.cherryq_scratch_bytes(16, k, n, c)
    ws_b, sc_b = lib.cherryq_workspace_bytes(rows, k, n, c), lib.cherryq_scratch_bytes(rows, k, n, c)
    assert sc_b > small_sc and ws_b >= small_ws
    ws = torch.zeros(ws_b, dtype=torch.uint8, device="cuda")
    sc = torch.empty(sc_b, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def call(scratch_bytes):
        return lib.cherryq_vecquant4matmul_f16(x.data_ptr(), d["qweight"].data_ptr(), d["cherry_weight"].data_ptr(),
                                               d["cherry_indices"].data_ptr(), d["scales"].data_ptr(), out.data_ptr(),
                                               rows, k, n, c, 128, 0, ws.data_ptr(), ws_b, sc.data_ptr(),
                                               scratch_bytes, stream)
    assert call(small_sc) == -4
    torch.cuda.synchronize()
    assert bool((out == 5.0).all())
    assert call(sc_b) == 0
    torch.cuda.synchronize()
    cols, sub = column_sample(p, np.random.default_rng(0), 256)
    assert orc.rel_l2(out.cpu().numpy()[:, cols], c_oracle.fused(x.cpu().numpy(), sub, bits, 128)) <= TOL
    assert not ws.any()   # the workspace is left zeroed


def test_empty_batch_is_a_no_op(qc):
    """Zero activation rows: nothing is launched, through the entry point and through the module."""
    announce("empty batch")
    from llama.qlinear import QuantLinear as PackedLinear
    from llama.quantizer import FullSymQuantizer
    k, n = 1024, 256
    p = orc.synthetic_packed_fast(k, n, 4, 128, seed=3)
    d = dev(p)
    x = torch.zeros(0, k, dtype=torch.float16, device="cuda")
    out = torch.zeros(0, n, dtype=torch.float16, device="cuda")
    qc.vecquant4matmul_cherryq(x, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], out, 128)
    q = PackedLinear(4, 128, FullSymQuantizer, 1 / 256, k, n, bias=False)
    for name in NAMES:
        setattr(q, name, d[name])
    y = q(torch.zeros(2, 0, k, dtype=torch.float16, device="cuda"))
    assert y.shape == (2, 0, n)
    torch.cuda.synchronize()
