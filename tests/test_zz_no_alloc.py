"""cherryq_vecquant_matmul_f16_static -- the entry point that allocates nothing (its split-K
accumulators live in a fixed array inside the library) -- called through the C ABI with raw
pointers and checked bit for bit against cherryq_vecquant{3,4}matmul_f16 with a caller's workspace
(same kernels, order-independent fixed-point accumulation): two calls in a row, the second with a
smaller input, so that whatever the first left in the shared array would show."""
import sys

import numpy as np
import pytest
import torch

from oracle import cherryq_oracle as orc
from oracle import c_oracle

pytestmark = pytest.mark.gpu


def _dev(p):
    return {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in p.items()
            if k in ("cherry_indices", "cherry_weight", "qweight", "scales")}


def _both(qc, bits, x, d, k, n, c, accumulate, base):
    """(static entry point's result, workspace entry point's result) for the same call."""
    lib = qc._lib
    b = x.shape[0]
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (True, False):
        out = base.clone()
        if static:
            rc = lib.cherryq_vecquant_matmul_f16_static(bits, x.data_ptr(), d["qweight"].data_ptr(),
                                                        d["cherry_weight"].data_ptr(), d["cherry_indices"].data_ptr(),
                                                        d["scales"].data_ptr(), out.data_ptr(), b, k, n, c, 128,
                                                        accumulate, stream)
        else:
            fn = lib.cherryq_vecquant4matmul_f16 if bits == 4 else lib.cherryq_vecquant3matmul_f16
            wsb = lib.cherryq_workspace_bytes(b, k, n, c)
            scb = lib.cherryq_scratch_bytes(b, k, n, c)
            ws = torch.zeros(wsb, dtype=torch.uint8, device="cuda")
            sc = torch.zeros(max(scb, 256), dtype=torch.uint8, device="cuda")
            rc = fn(x.data_ptr(), d["qweight"].data_ptr(), d["cherry_weight"].data_ptr(), d["cherry_indices"].data_ptr(),
                    d["scales"].data_ptr(), out.data_ptr(), b, k, n, c, 128, accumulate, ws.data_ptr(), wsb,
                    sc.data_ptr(), sc.numel(), stream)
        assert rc == 0, (static, rc)
        torch.cuda.synchronize()
        outs.append(out)
    return outs


@pytest.mark.parametrize("bits", [4, 3])
def test_static_workspace_entry_point_matches_the_workspace_one(bits):
    assert torch.cuda.is_available()
    import quant_cuda as qc
    print("[case] static-workspace entry point", bits, flush=True)
    sys.stdout.flush()
    rng = np.random.default_rng(21 + bits)
    layers = {}
    # first a larger call (2 rows, 4096 -> 11008), then smaller ones (1 row 4096 -> 4096; 4 rows 1024 -> 520)
    for (k, n, b, accumulate) in ((4096, 11008, 2, 0), (4096, 4096, 1, 1), (1024, 520, 4, 0), (4096, 11008, 1, 0)):
        if (k, n) not in layers:
            layers[(k, n)] = orc.synthetic_layer(k, n, bits, 128, seed=30)[1]
        p = layers[(k, n)]
        d = _dev(p)
        c = int(p["cherry_indices"].shape[0])
        xh = rng.standard_normal((b, k)).astype(np.float16)
        x = torch.from_numpy(xh).cuda()
        base = torch.from_numpy(rng.standard_normal((b, n)).astype(np.float16)).cuda()
        got, want = _both(qc, bits, x, d, k, n, c, accumulate, base)
        assert torch.equal(got, want), (k, n, b, accumulate)
        ref = c_oracle.fused(xh, p, bits, 128) + (base.cpu().numpy().astype(np.float64) if accumulate else 0.0)
        assert orc.rel_l2(got.cpu().numpy(), ref) <= 1e-3, (k, n, b)
    # the python wrapper takes the same route
    out = torch.empty(b, n, dtype=torch.float16, device="cuda")
    qc.matmul_cherryq_static(bits, x, d["qweight"], d["cherry_weight"], d["cherry_indices"], d["scales"], out, 128)
    torch.cuda.synchronize()
    assert torch.equal(out, want)


def test_static_workspace_entry_point_rejects_what_exceeds_its_array():
    import quant_cuda as qc
    lib = qc._lib
    fake = 1 << 12
    args = lambda bits, b, k, n, c, g: (bits, fake, fake, fake, fake, fake, fake, b, k, n, c, g, 0, None)
    assert lib.cherryq_vecquant_matmul_f16_static(*args(4, 5, 4096, 4096, 16, 128)) == -8       # more than 4 rows
    assert lib.cherryq_vecquant_matmul_f16_static(*args(4, 4, 4096, 32776, 16, 128)) == -8      # 4 x 32776 words
    assert lib.cherryq_vecquant_matmul_f16_static(*args(3, 1, 4096, 131080, 16, 128)) == -8
    assert lib.cherryq_vecquant_matmul_f16_static(*args(5, 1, 4096, 4096, 16, 128)) == -5
    assert lib.cherryq_vecquant_matmul_f16_static(*args(4, 1, 4096, 4096, 16, 64)) == -3
    assert lib.cherryq_vecquant_matmul_f16_static(*args(4, 1, 4096, 4100, 16, 128)) == -2
    assert b"fixed workspace" in lib.cherryq_status_string(-8)
