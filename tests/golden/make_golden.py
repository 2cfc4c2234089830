"""Writes the golden fixtures in this directory from the reference's own Python.

Run once, in the build container (the reference is mounted read-only there):

    python tests/golden/make_golden.py [/root/reference]

It imports the reference's pure-torch modules `llama.quantizer`, `llama.cherry_linear`
and `llama.qlinear` on the CPU and records input/output vectors of

  * FullSymQuantizer.get_scaling_factor / quantize / dequantize / transform,
  * cherry_linear.QuantLinear._get_scaling_factors / _adjust_weight,
  * qlinear.QuantLinear.pack / unpack / forward under dmode(layerwise_dequantize=False),

for small layers (3- and 4-bit, group 128 / 64 / -1, fp16 and fp32 weights).  The fused
entry points of the reference need its compiled extension, which cannot be built here;
`llama.qlinear` imports that extension by name at module import, so an empty module
object of that name is registered first -- none of the recorded functions calls into it.

Only data is written: `golden_<case>.npz` files loadable with numpy.load (no pickle).
"""
import sys
import types
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent

CASES = [
    # name, w_bits, group_size, in, out, cherry_fraction, weight dtype, seed
    ("w4_g128_k256", 4, 128, 256, 16, 1 / 16, torch.float16, 1),
    ("w3_g128_k256", 3, 128, 256, 16, 1 / 16, torch.float16, 2),
    ("w4_g128_k2048", 4, 128, 2048, 24, 1 / 256, torch.float16, 3),
    ("w3_g128_k2048", 3, 128, 2048, 24, 1 / 256, torch.float16, 4),
    ("w3_g64_k256", 3, 64, 256, 16, 1 / 16, torch.float16, 5),
    ("w4_gall_k256", 4, -1, 256, 8, 1 / 32, torch.float16, 6),
    ("w4_g128_k512_f32", 4, 128, 512, 8, 1 / 32, torch.float32, 7),
    ("w3_g128_k512_f32", 3, 128, 512, 8, 1 / 32, torch.float32, 8),
    ("w4_g128_k128_nocherry", 4, 128, 128, 8, 1 / 256, torch.float16, 9),
]


def make_weight(n, k, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.02
    mask = torch.rand(n, k, generator=g) < 0.01
    w = torch.where(mask, w * 10, w)
    # rows that exercise edges: an all-zero group, exact grid ties, a huge outlier
    w[0, : min(k, 128)] = 0.0
    if n > 1:
        w[1, :8] = torch.tensor([0.5, 1.0, 1.5, 2.0, 2.5, 3.0, 3.5, 4.0]) * 0.125
    if n > 2:
        w[2, 5] = 3.0
    return w.to(dtype)


def main(ref_root):
    sys.path.insert(0, ref_root)
    sys.modules.setdefault("quant_cuda", types.ModuleType("quant_cuda"))
    from llama.quantizer import FullSymQuantizer
    from llama.cherry_linear import QuantLinear as TrainLinear
    from llama.qlinear import QuantLinear as PackedLinear

    torch.set_grad_enabled(False)
    for name, bits, gs, k, n, frac, dtype, seed in CASES:
        w = make_weight(n, k, dtype, seed)
        lin = TrainLinear(k, n, bias=False, w_bits=bits, group_size=gs if gs != -1 else k,
                          cherryq=True, cherry_fraction=frac)
        lin = lin.to(dtype)
        lin.weight.data.copy_(w)
        lin.eval()
        c = lin.num_cherries
        g = torch.Generator().manual_seed(seed + 100)
        score = w.float().abs().amax(0)
        idx = torch.argsort(score, descending=True, stable=True)[:c]
        idx = idx[torch.randperm(c, generator=g)]  # unsorted on purpose: pack() sorts
        lin.register_cherry_indices(idx)

        out = {"weight": w.numpy(), "cherry_indices_in": idx.numpy().astype(np.int32),
               "meta": np.array([bits, gs, k, n, c], dtype=np.int64),
               "cherry_fraction": np.array([frac])}

        # quantiser functions on the first group of the compacted normal weight
        mask = torch.ones(k, dtype=torch.bool)
        mask[idx] = False
        nw = w[:, mask.nonzero().squeeze(1)]
        geff = gs if gs != -1 else k
        grp = nw[:, :geff]
        s = FullSymQuantizer.get_scaling_factor(grp, None, bits, False)
        out["q_group"] = grp.numpy()
        out["q_scale"] = s.numpy()
        out["q_quantize"] = FullSymQuantizer.quantize(grp, s, bits).numpy()
        out["q_dequantize"] = FullSymQuantizer.dequantize(
            FullSymQuantizer.quantize(grp, s, bits).to(torch.int8), s).numpy()
        out["q_transform"] = FullSymQuantizer.transform(grp, s, bits).numpy()

        out["scaling_factors"] = lin._get_scaling_factors(nw).numpy()
        out["adjust_weight"] = lin._adjust_weight(w.clone(), ste=False).numpy()

        q = PackedLinear(bits, gs, lin.quantizer, frac, k, n, bias=False)
        q.pack(lin)
        out["cherry_indices"] = q.cherry_indices.numpy()
        out["cherry_weight"] = q.cherry_weight.numpy()
        out["qweight"] = q.qweight.numpy()
        out["scales"] = q.scales.numpy()
        dense = q.unpack()
        out["unpack"] = dense.numpy()

        x = torch.randn(3, k, generator=g).to(torch.float16)
        out["x"] = x.numpy()
        with PackedLinear.dmode(layerwise_dequantize=False):
            y = q(x)
        out["forward_dequantized"] = y.numpy()

        path = HERE / f"golden_{name}.npz"
        np.savez_compressed(path, **out)
        print(f"wrote {path.name}: " + ", ".join(f"{a}{tuple(v.shape)}" for a, v in out.items()))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
