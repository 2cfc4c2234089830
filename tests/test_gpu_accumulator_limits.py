"""The split-K accumulator's contract at its limits.  fp16 tensors: partial sums are carried as
multiples of 2^-34 within +-2^21 -- large partials that cancel across workgroups come out exact,
results beyond fp16's range come out as infinities of the right sign, and (documented, not desired)
a NaN activation reads as a partial at the end of the range: infinite outputs, not NaN.  fp32 tensors: partials outside that range take a
float side accumulator, so results beyond 2^21, infinities and NaN behave as in fp32."""
import sys

import numpy as np
import pytest
import torch

from oracle import cherryq_oracle as orc
from oracle import c_oracle

pytestmark = pytest.mark.gpu
NAMES = ("cherry_indices", "cherry_weight", "qweight", "scales")


def _fused16(qc, bits, x, p):
    d = {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in p.items() if k in NAMES}
    out = torch.zeros(x.shape[0], p["qweight"].shape[1], dtype=torch.float16, device="cuda")
    qc.matmul_cherryq(bits, torch.from_numpy(x).cuda(), d["qweight"], d["cherry_weight"], d["cherry_indices"],
                      d["scales"], out, 128)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("bits", [4, 3])
@pytest.mark.parametrize("rows", [1, 2, 4])
def test_fp16_large_cancelling_partials_and_overflow_sign(bits, rows):
    import quant_cuda as qc
    print("[case] accumulator limits fp16", bits, rows, flush=True)
    sys.stdout.flush()
    k, n = 4096, 1024
    p = dict(orc.synthetic_layer(k, n, bits, 128, seed=40 + bits)[1])
    # weights 2^10 times larger (exact in fp16): |w| up to a few tens
    p["scales"] = (p["scales"].astype(np.float32) * 1024).astype(np.float16)
    p["cherry_weight"] = (p["cherry_weight"].astype(np.float32) * 1024).astype(np.float16)
    wmax = float((2 ** bits - 1) / 2 * p["scales"].astype(np.float64).max())   # of the quantised columns, the only ones hit
    amp = 2.0 ** np.floor(np.log2(2.0 ** 19 / wmax))          # every single product stays below 2^19
    nidx = orc.normal_indices(k, p["cherry_indices"].astype(np.int64))
    x = np.zeros((rows, k), dtype=np.float16)
    for r in range(rows):
        # two huge activations of opposite sign in different workgroups' K ranges, one ordinary one
        x[r, nidx[5 + r]] = amp
        x[r, nidx[5 + r + 2048]] = -amp
        x[r, nidx[1000 + r]] = 1.0
    want64 = c_oracle.fused(x, p, bits, 128)
    assert np.abs(want64).max() < 2.0 ** 21 and np.abs(want64).max() > 65520   # inside the contract, beyond fp16
    with np.errstate(over="ignore"):
        want = want64.astype(np.float16)
    got = _fused16(qc, bits, x, p)
    assert np.isinf(want).any() and np.isfinite(want).any()
    np.testing.assert_array_equal(got, want)   # exact finite values, +inf / -inf where fp16 overflows


def test_fp16_nan_activation_gives_non_finite_outputs():
    """Documented limitation of the fixed-point accumulator: a NaN partial cannot be carried; it is
    clamped like any out-of-range value (to +-2^21), so the outputs are infinities (of either sign)
    instead of NaN -- still not finite -- and the workspace is left clean (the next call is right)."""
    import quant_cuda as qc
    print("[case] accumulator NaN fp16", flush=True)
    k, n = 4096, 512
    p = orc.synthetic_layer(k, n, 4, 128, seed=44)[1]
    x = np.random.default_rng(2).standard_normal((1, k)).astype(np.float16)
    clean = _fused16(qc, 4, x, p)
    bad = x.copy()
    bad[0, 77] = np.nan
    got = _fused16(qc, 4, bad, p)
    assert not np.isfinite(got).any()
    np.testing.assert_array_equal(_fused16(qc, 4, x, p), clean)


@pytest.mark.parametrize("b,g", [(1, 128), (4, 128), (16, 128), (3, 64)])
def test_fp32_results_beyond_the_fixed_point_range_and_non_finite_values(b, g):
    """(b, g) pick the kernels: one row without scratch and group 64 run the general kernel, the
    others the matrix-core one."""
    import quant_cuda as qc
    print("[case] accumulator limits fp32", b, g, flush=True)
    k, n, c = 2048, 512, 8
    kn = k - c
    rng = np.random.default_rng(50 + b)
    qweight = rng.integers(0, 256, size=(kn // 8 * 3, n), dtype=np.uint8)
    cw = rng.standard_normal((c, n)).astype(np.float32)
    idx = np.sort(rng.choice(k, c, replace=False)).astype(np.int32)
    scales = (rng.random((-(-kn // g), n)) * 0.01 + 0.005).astype(np.float32)
    u = orc.unpack_codes(qweight, 3).astype(np.float64) - 3.5
    wn = u * np.repeat(scales.astype(np.float64), g, axis=0)[:kn]
    nidx = orc.normal_indices(k, idx)
    t = [torch.from_numpy(a).cuda() for a in (qweight, cw, idx, scales)]

    def run(vec):
        mul = torch.zeros(b, n, device="cuda")
        qc.vecquant3matmul_cherryq(torch.from_numpy(vec).cuda(), *t, mul, g, False)
        torch.cuda.synchronize()
        return mul.cpu().numpy()

    def want(vec):
        return vec[:, nidx].astype(np.float64) @ wn + vec[:, idx].astype(np.float64) @ cw.astype(np.float64)

    base = rng.standard_normal((b, k)).astype(np.float32)
    # rows of very different magnitude: row 0 ordinary, the others scaled up to 1e12
    big = base * np.logspace(0, 12, b, dtype=np.float64)[:, None].astype(np.float32) if b > 1 else base * np.float32(1e9)
    got, ref = run(big), want(big)
    assert np.abs(ref).max() > 2.0 ** 21
    for r in range(b):
        tol = 2e-6 * np.abs(ref[r]).max() * np.sqrt(k / 1024) + 2.0 ** -30
        assert np.abs(got[r] - ref[r]).max() <= tol, r
    # infinities and NaN arrive where fp32 arithmetic puts them; other rows are untouched
    special = base.copy()
    special[0, int(nidx[3])] = np.inf
    got = run(special)
    col_sign = np.sign(wn[3])
    assert np.all(np.isinf(got[0][col_sign != 0])) and np.all(np.sign(got[0][col_sign != 0]) == col_sign[col_sign != 0])
    special[0, int(nidx[900])] = np.nan
    got = run(special)
    assert np.all(np.isnan(got[0]))
    if b > 1:
        ref = want(base)
        assert np.abs(got[1:] - ref[1:]).max() <= 2e-6 * np.abs(ref).max() * np.sqrt(k / 1024)
    # the workspace (words and side accumulators) is clean again
    got, ref = run(base), want(base)
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max() * np.sqrt(k / 1024)
