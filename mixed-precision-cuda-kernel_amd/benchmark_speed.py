"""Operator micro-benchmark with the call shapes of the reference's benchmark_speed.py:20-45:
3-bit, batch 16, 4096 -> 13824, group 128, 16 cherry channels, `mul` accumulated into 100 times;
the fp32 variant (fp32 tensors, int32 indices) the reference times, the fp16 variant its model
uses (llama/qlinear.py:168-181), and a dense fp16 matmul of the same shape beside them.

    python mixed-precision-cuda-kernel_amd/benchmark_speed.py          (needs the MI355X)
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import torch

import quant_cuda


def timed(name, fn, reps=100):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    print(f"{name:44s} {e0.elapsed_time(e1) * 1e3 / reps:9.1f} us per call")


def main():
    torch.manual_seed(0)
    batch, k, n, c, group = 16, 4096, 13824, 16, 128
    kn = k - c
    vec = torch.randn(batch, k, device="cuda")
    qweight = torch.randint(0, 256, (kn // 8 * 3, n), dtype=torch.uint8, device="cuda")
    cherry_weight = torch.randn(c, n, device="cuda")
    cherry_indices = torch.randperm(k, device="cuda")[:c].sort().values.to(torch.int32)
    scales = torch.rand(-(-kn // group), n, device="cuda") * 0.01 + 0.005
    mul = torch.zeros(batch, n, device="cuda")
    weight_half = torch.randn(k, n, device="cuda").half()
    vec_h, cw_h, sc_h = vec.half(), cherry_weight.half(), scales.half()
    idx_h, mul_h = cherry_indices.to(torch.int16), torch.zeros(batch, n, dtype=torch.float16, device="cuda")

    timed("dense fp16 matmul (16 x 4096 x 13824)", lambda: torch.matmul(vec_h, weight_half))
    timed("vecquant3matmul_cherryq fp32, batch 16",
          lambda: quant_cuda.vecquant3matmul_cherryq(vec, qweight, cherry_weight, cherry_indices, scales, mul, group, False))
    timed("vecquant3matmul_cherryq fp16, batch 16",
          lambda: quant_cuda.vecquant3matmul_cherryq(vec_h, qweight, cw_h, idx_h, sc_h, mul_h, group, True))
    timed("vecquant3matmul_cherryq fp16, batch 1",
          lambda: quant_cuda.vecquant3matmul_cherryq(vec_h[:1], qweight, cw_h, idx_h, sc_h, mul_h[:1], group, True))


if __name__ == "__main__":
    main()
