"""Benchmark of the CherryQ hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all]

A step is one fused CherryLinear matvec (batch 1) over one packed layer resident in HBM.  The
default workload is the headline configuration: LLaMA-7B gate/up shape 4096 -> 11008, 4-bit,
group 128, 1/256 cherry channels.  Every step uses a different copy of the packed layer, cycling
through enough copies (> 512 MB) that nothing is served from the 256 MB Infinity Cache.

Prints one JSON line:  metric = microseconds per matvec (whole-job, HIP events around the K
timed launches on the launch stream);  roofline = algorithmic bytes per launch / that time,
against the 8 TB/s HBM peak;  cpu_baseline = the reference's CPU path (unpack + linear) as
restated by the C oracle, timed on this host.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (str(ROOT), str(ROOT / "mixed-precision-cuda-kernel_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (w_bits, in_features, out_features)
    "llama7b_gate_up_w4": (4, 4096, 11008),
    "llama7b_gate_up_w3": (3, 4096, 11008),
    "llama7b_down_w4": (4, 11008, 4096),
    "llama7b_down_w3": (3, 11008, 4096),
    "llama7b_attn_w4": (4, 4096, 4096),
    "llama7b_attn_w3": (3, 4096, 4096),
    "llama13b_attn_w3": (3, 5120, 5120),
    "llama13b_gate_up_w3": (3, 5120, 13824),
    "llama13b_down_w3": (3, 13824, 5120),
    "llama70b_attn_w4": (4, 8192, 8192),
    "llama70b_kv_w4": (4, 8192, 1024),
    "llama70b_gate_up_w4": (4, 8192, 28672),
    "llama70b_down_w4": (4, 28672, 8192),
}


# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, each
# counter scaled by its reading for a 256 MiB device copy (x2.000 and x1.000); the counters
# cannot be read while timing, so the figure is recorded here for the workloads measured.
MEASURED_TRAFFIC = {("llama7b_gate_up_w4", 1, "reference"): 25320960,
                    ("llama7b_gate_up_w4", 1, "prepacked"): 23834070}


# Matrix-core busy share of the 8- and 16-row kernels from rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES runs (busy
# cycles / (kernel time x 2.4 GHz x 1024 SIMDs)); like the traffic figure it cannot be read while timing.
MFMA_BUSY = {("llama13b_gate_up_w3", 8): {"frac": 0.092, "kernel": "cq::stream_cu_rows_kernel<3, 4, 12, 3, 4, 3, 3, 4, 8>",
                                          "profile": "profiles/stream_cu_rows_w3_w4_llama13b_llama7b_gate_up_rows4_rows8.md"},
             ("llama13b_attn_w3", 8): {"frac": 0.057, "kernel": "cq::stream_cu_rows_kernel<3, 5, 8, 2, 6, 2, 3, 4, 8>",
                                       "profile": "profiles/stream_cu_rows_w3_w4_llama13b_llama7b_gate_up_rows4_rows8.md"},
             "llama70b_gate_up_w4": {"frac": 0.123, "kernel": "cq::stream_rows_reg_kernel<4, 8, 8, 1>",
                                     "profile": "profiles/rows16_w4_llama70b_gate_up_8192x28672_stream.md"},
             "llama70b_down_w4": {"frac": 0.135, "kernel": "cq::stream_rows_reg_kernel<4, 8, 8, 1, true>",
                                  "profile": "profiles/rows16_w4_llama70b_down_28672x8192_stream.md"}}


def algorithmic_bytes(bits, k, n, batch=1, group=128):
    """Bytes one call must move: packed codes + scales + cherry rows + indices + x + y."""
    c = -(-k // 256) // 8 * 8
    kn = k - c
    return kn // 8 * bits * n + -(-kn // group) * n * 2 + c * n * 2 + c * 2 + batch * k * 2 + batch * n * 2


def make_copies(bits, k, n, group, min_bytes, seed=0):
    """Distinct packed layers (uniform random codes, scales such that the dequantised weights
    have a standard deviation near 0.02, sorted random cherry channels with N(0, 0.02) fp16
    weights) totalling > min_bytes on the GPU.  Returns (copy 0 as numpy arrays, list of copies)."""
    import math
    import torch
    c = -(-k // 256) // 8 * 8
    kn = k - c
    g = torch.Generator(device="cuda").manual_seed(seed)
    code_std = math.sqrt((4 ** bits - 1) / 12.0)
    first = {
        "qweight": torch.randint(0, 256, (kn // 8 * bits, n), dtype=torch.uint8, device="cuda", generator=g),
        "scales": ((torch.rand((-(-kn // group), n), device="cuda", generator=g) * 0.5 + 0.75)
                   * (0.02 / code_std)).half(),
        "cherry_weight": (torch.randn((c, n), device="cuda", generator=g) * 0.02).half(),
        "cherry_indices": torch.randperm(k, device="cuda", generator=g)[:c].sort().values.to(torch.int16),
    }
    per = sum(v.numel() * v.element_size() for v in first.values())
    ncopies = max(2, -(-min_bytes // per))
    copies = [first]
    for i in range(1, ncopies):
        t = dict(first)
        t["qweight"] = torch.randint(0, 256, first["qweight"].shape, dtype=torch.uint8, device="cuda", generator=g)
        copies.append(t)
    base = {name: v.cpu().numpy() for name, v in first.items()}
    return base, copies


def _replays(steps):
    """How many times the K-step sequence is repeated INSIDE the captured graph: enough that a short
    run (the driver's --steps 20) is timed over about 2000 back-to-back launches, like a long one.
    (Replaying a 20-launch graph 100 times instead read 0.5 us per launch higher: every replay
    boundary costs about 10 us of launch latency that a serving loop's long graph does not pay.)"""
    return max(1, -(-2000 // max(1, steps)))


TIMED_REPLAYS = 5


def _time_graph(stream, build, steps):
    """Capture steps * _replays(steps) launches (build(i) enqueues launch i) into ONE HIP graph,
    replay it TIMED_REPLAYS times with a HIP event before and after each replay (recorded on the
    launch stream) and return the MEDIAN replay's microseconds per launch.  One untimed replay first."""
    import torch
    total = steps * _replays(steps)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for i in range(total):
            build(i)
    graph.replay()
    stream.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(TIMED_REPLAYS + 1)]
    ev[0].record(stream)
    for j in range(TIMED_REPLAYS):
        graph.replay()
        ev[j + 1].record(stream)
    stream.synchronize()
    per = sorted(ev[j].elapsed_time(ev[j + 1]) * 1e3 / total for j in range(TIMED_REPLAYS))
    return per[len(per) // 2]


def time_gpu(bits, k, n, group, steps, warmup, batch=1, use_graph=True, path="auto"):
    """Device time per fused call.  The `steps` launches (each on a different copy of the packed
    layer) are captured once into a HIP graph and replayed, so the figure is the GPU's launch-to-
    launch time and not the Python binding's; HIP events bracket every replay on the launch stream.
    path: "reference" = the kernels that read the checkpoint layout, "prepacked" = the load-time
    repacked weight stream (batch 1), "auto" = what a loader gets: prepacked where the library
    recommends it for the shape (quant_cuda.prepack_recommended).
    Returns a dict (us, path, eager host wall us, cache-resident us, first copy as numpy, ...)."""
    import numpy as np
    import torch
    import quant_cuda
    base, copies = make_copies(bits, k, n, group, 640 << 20)
    c = copies[0]["cherry_indices"].numel()
    if path == "auto":
        path = "prepacked" if (quant_cuda.prepack_recommended(bits, k, n, c, group) and
                               (batch == 1 or (batch <= 16 and quant_cuda.prepacked_rows_recommended(bits, batch, k, n, c, group)))) \
            else "reference"
    x = torch.from_numpy(np.random.default_rng(1).standard_normal((batch, k)).astype(np.float16)).cuda()
    out = torch.zeros(batch, n, dtype=torch.float16, device="cuda")
    if path == "prepacked":
        for t in copies:
            t["stream"] = quant_cuda.prepack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"],
                                                     t["scales"], k, group)
            del t["qweight"]  # the 29 reference-layout copies are not needed any more
        torch.cuda.empty_cache()

    def step(i):
        t = copies[i % len(copies)]
        if path == "prepacked":
            quant_cuda.matvec_prepacked_cherryq(bits, x, t["stream"], out, k, c)
        else:
            quant_cuda.matmul_cherryq(bits, x, t["qweight"], t["cherry_weight"], t["cherry_indices"], t["scales"], out,
                                      group, accumulate=False)

    stream = torch.cuda.Stream()
    res = {"path": path, "base": base, "x": x, "out": out, "copies": copies, "resident_us": None}
    with torch.cuda.stream(stream):
        # eager: untimed warm-up, then the host-inclusive rate
        for i in range(warmup):
            step(i)
        stream.synchronize()
        t0 = time.perf_counter()
        for i in range(min(steps, 500)):
            step(warmup + i)
        stream.synchronize()
        res["wall_us"] = (time.perf_counter() - t0) * 1e6 / min(steps, 500)
        if use_graph:
            res["us"] = _time_graph(stream, lambda i: step(warmup + i), steps)
            # the same launches on ONE copy: the packed layer then comes from the Infinity Cache
            # (reported beside the HBM figure, labelled; it is never the headline value)
            res["resident_us"] = _time_graph(stream, lambda i: step(0), steps)
        else:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for i in range(steps):
                step(warmup + i)
            e1.record(stream)
            stream.synchronize()
            res["us"] = e0.elapsed_time(e1) * 1e3 / steps
    return res


def roofline_reference(nbytes, steps):
    """What the GPU does with the same number of bytes when a kernel only reads them, and what an
    empty launch costs (libcherryq_probe.so, a bench-only library): the plain read is swept over
    8 / 16 / 32 / 64 KB per workgroup and the read-once / default cache policy, same rotation over
    > 512 MB, same graph replays; the fastest is reported.  Puts the fused kernel's time in proportion."""
    import ctypes
    import torch
    lib = ctypes.CDLL(str(ROOT / "mixed-precision-cuda-kernel_amd" / "libcherryq_probe.so"))
    lib.cherryq_probe_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int,
                                              ctypes.c_int, ctypes.c_void_p]
    lib.cherryq_probe_empty_launch.argtypes = [ctypes.c_void_p]
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    per = (nbytes + 4095) // 4096 * 4096
    ncopies = max(2, -(-(640 << 20) // per))
    buf = torch.randint(0, 256, (per * ncopies,), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.Stream()
    sweep = {}
    with torch.cuda.stream(stream):
        def timed(fn):
            for i in range(20):
                fn(i)
            stream.synchronize()
            return _time_graph(stream, fn, steps)

        for kb in (8, 16, 32, 64):
            for nt in (1, 0):
                def read(i, kb=kb, nt=nt):
                    rc = lib.cherryq_probe_stream_read(buf.data_ptr() + (i % ncopies) * per, nbytes, sink.data_ptr(), kb, nt,
                                                       stream.cuda_stream)
                    assert rc == 0, rc
                sweep[f"{kb}KB{'_nt' if nt else ''}"] = round(timed(read), 3)

        def empty(i):
            assert lib.cherryq_probe_empty_launch(stream.cuda_stream) == 0
        empty_us = timed(empty)
    best = min(sweep, key=sweep.get)
    del buf
    torch.cuda.empty_cache()
    return {"plain_read_us": sweep[best], "plain_read_shape": best, "plain_read_bytes": nbytes,
            "plain_read_gbs": round(nbytes / sweep[best] / 1e3, 1), "plain_read_sweep_us": sweep,
            "empty_launch_us": round(empty_us, 3)}


def cpu_baseline(bits, k, n, group, base, x_np, seconds=8.0):
    """The reference CPU path -- QuantLinear.unpack() then linear -- restated in C (oracle),
    timed on this host: cold = unpack + matvec, cached = matvec on the dense fp16 weight."""
    import numpy as np
    from oracle import c_oracle
    threads = c_oracle.threads()
    dense = np.zeros((n, k), dtype=np.float16)
    c_oracle.dequant_matmul(x_np, base, bits, group, dense)  # warm-up
    reps, cold = 0, []
    t_end = time.perf_counter() + seconds
    while reps < 3 or time.perf_counter() < t_end:  # a bounded sample: `seconds` of wall time on all host threads
        t0 = time.perf_counter()
        c_oracle.dequant_matmul(x_np, base, bits, group, dense)
        cold.append(time.perf_counter() - t0)
        reps += 1
    cached = []
    for _ in range(min(max(3, reps), 200)):
        t0 = time.perf_counter()
        c_oracle.linear(x_np, dense)
        cached.append(time.perf_counter() - t0)
    cold_us = float(np.median(cold)) * 1e6
    return {"value": round(cold_us, 1), "unit": "us/matvec", "cores": threads, "kind": "port",
            "sample": f"{reps} calls of unpack()+linear on the same {k}x{n} {bits}-bit layer, median; "
                      f"cached dense fp16 linear alone: {float(np.median(cached)) * 1e6:.1f} us"}


def decode_benchmark(prompt_len=128, new_tokens=128, w_bits=4, seed=0):
    """Random-init LLaMA-7B-shape decoder (32 layers, hidden 4096, 32 heads,
    MLP 11008, vocab 32000, all seven linears per layer 4-bit CherryLinear, group 128, 1/256
    cherries), greedy decoding at batch 1: 128 random prompt ids, then 128 generated tokens.
    The token step is one captured HIP graph; decode tokens/s excludes the prompt."""
    import numpy as np
    import torch
    import cherryq_decoder as cd
    cfg = cd.DecoderConfig(w_bits=w_bits, max_position_embeddings=prompt_len + new_tokens)
    model = cd.CherryLlamaDecoder(cfg, seed=seed)
    prompt = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=torch.Generator().manual_seed(seed))
    # first on the checkpoint layout alone, then as a loader leaves the model: the layers the
    # library recommends it for repacked into weight streams
    model.capture(fork=False)
    model.generate(prompt, 8)
    _, _, ref_total = model.generate(prompt, new_tokens)
    repacked = model.prepack()
    model.capture(fork=False)
    model.generate(prompt, 8)                                   # warm-up
    out, _, total = model.generate(prompt, new_tokens)          # throughput: one sync at the end
    _, times, _ = model.generate(prompt, new_tokens, sync_each_token=True)  # latency per token
    # prompt processing: token by token through the captured step, and in one batched pass
    def timed(fn, reps=3):
        best = float("inf")
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t0)
        return best
    model.prefill(prompt)                                        # warm-up (workspaces for 128 rows)
    prefill_batched = timed(lambda: model.prefill(prompt))
    prefill_steps = timed(lambda: model.generate(prompt, 0), reps=1)
    bytes_per_token = model.step_bytes()
    tok_s = new_tokens / total
    res = {"model": "llama7b-shape random init", "w_bits": w_bits, "prompt_tokens": prompt_len,
           "generated_tokens": new_tokens, "tokens_per_s": round(tok_s, 1),
           "ms_per_token_median_synced": round(float(np.median(times)) * 1e3, 4),
           "packed_bytes_per_token": bytes_per_token,
           "hbm_gbs": round(bytes_per_token * tok_s / 1e9, 1),
           "frac_of_hbm_peak": round(bytes_per_token * tok_s / 1e9 / HBM_PEAK_GBS, 4),
           "launch": "one single-stream HIP graph per token",
           "layers_repacked_at_load": repacked,
           "tokens_per_s_checkpoint_layout_only": round(new_tokens / ref_total, 1),
           "prefill_ms_batched": round(prefill_batched * 1e3, 2),
           "prefill_ms_token_steps": round(prefill_steps * 1e3, 2),
           "first_tokens": out[:8].tolist()}
    del model
    torch.cuda.empty_cache()
    return res


def unpack_table(group):
    """Dense dequantisation (QuantLinear.unpack on the GPU) of whole layers: device time per call
    and the bytes it moves (packed buffers read once, dense fp16 weight written once)."""
    import torch
    import quant_cuda
    for bits in (4, 3):
        for k, n in ((4096, 11008), (11008, 4096), (4096, 4096), (8192, 28672)):
            _, (t, _) = make_copies(bits, k, n, group, 0, seed=k + bits)
            fn = lambda: quant_cuda.unpack_cherryq(bits, t["qweight"], t["cherry_weight"], t["cherry_indices"],
                                                   t["scales"], k, group)
            for _ in range(3):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / 20 * 1e3
            ab = sum(v.numel() * v.element_size() for v in t.values()) + 2.0 * k * n
            print(f"unpack {bits}-bit {k:5d}->{n:5d}: {us:7.2f} us  {ab / us / 1e3:7.1f} GB/s "
                  f"({ab / us / 1e3 / HBM_PEAK_GBS * 100:4.1f}% of 8 TB/s; packed read + dense fp16 write)",
                  file=sys.stderr, flush=True)
            del t
            torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="llama7b_gate_up_w4", choices=sorted(WORKLOADS))
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--batch", type=int, default=1, help="activation rows per call (2..4: streaming kernel with several rows or, like 5..16, the small-batch matrix-core kernel; more: tiled GEMM kernel)")
    ap.add_argument("--all", action="store_true", help="also print a table of every workload to stderr")
    ap.add_argument("--unpack-only", action="store_true",
                    help="print the dense-dequantisation table to stderr and exit (for profiling that kernel)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the 7B-shape decode measurement")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a graph replay")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run 8 plain device copies of 256 MiB (a known-size kernel for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures the hot path on ONE GPU; --gpus N > 1 is not supported "
              "(the path shards by output columns without any exchange).", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)

    if args.calibrate_copy:
        src = torch.randint(0, 256, (256 << 20,), dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(8):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    if args.unpack_only:
        unpack_table(args.group)
        return
    if args.all:
        # the small-batch path (matrix cores) on the 13B and 70B layer shapes
        for name, b in (("llama7b_gate_up_w4", 2), ("llama7b_attn_w4", 2), ("llama7b_attn_w4", 4),
                        ("llama13b_attn_w3", 4), ("llama13b_attn_w3", 8), ("llama13b_gate_up_w3", 8),
                        ("llama13b_down_w3", 8), ("llama70b_attn_w4", 16), ("llama70b_kv_w4", 16),
                        ("llama70b_gate_up_w4", 16), ("llama70b_down_w4", 16), ("llama7b_gate_up_w4", 16)):
            bits, k, n = WORKLOADS[name]
            us = time_gpu(bits, k, n, args.group, max(200, args.steps // 4), args.warmup, batch=b,
                          use_graph=not args.no_graph)["us"]
            ab = algorithmic_bytes(bits, k, n, b, args.group)
            fl = 2.0 * b * k * n
            print(f"{name:24s} {bits}-bit {k:5d}->{n:5d} batch {b:2d}: {us:7.2f} us  {ab / us / 1e3:7.1f} GB/s "
                  f"{ab / us / 1e3 / HBM_PEAK_GBS * 100:5.1f}% of 8 TB/s  {fl / us / 1e6:6.1f} TFLOP/s "
                  f"({fl / us / 1e6 / 2500 * 100:4.1f}% of fp16 MFMA peak; whole call)",
                  file=sys.stderr, flush=True)
            torch.cuda.empty_cache()
        # prompt-sized batches: the tiled dequantise + MFMA GEMM kernel
        for name, b in (("llama7b_attn_w4", 128), ("llama7b_gate_up_w4", 32), ("llama7b_gate_up_w4", 128),
                        ("llama7b_gate_up_w3", 128), ("llama7b_down_w4", 128), ("llama7b_gate_up_w4", 512),
                        ("llama7b_gate_up_w4", 2048), ("llama70b_gate_up_w4", 128), ("llama70b_down_w4", 128)):
            bits, k, n = WORKLOADS[name]
            us = time_gpu(bits, k, n, args.group, 100, 10, batch=b, use_graph=not args.no_graph)["us"]
            ab = algorithmic_bytes(bits, k, n, b, args.group)
            fl = 2.0 * b * k * n
            print(f"{name:24s} {bits}-bit {k:5d}->{n:5d} rows {b:4d}: {us:7.2f} us  {fl / us / 1e6:6.1f} TFLOP/s "
                  f"({fl / us / 1e6 / 2500 * 100:4.1f}% of fp16 MFMA peak)  {ab / us / 1e3:7.1f} GB/s "
                  f"({ab / us / 1e3 / HBM_PEAK_GBS * 100:4.1f}% of 8 TB/s; prep + main kernel)",
                  file=sys.stderr, flush=True)
            torch.cuda.empty_cache()
        # training side: the fused fake quantisation of a whole weight, against the torch operations it replaces
        import quant_cuda
        from llama.cherry_linear import QuantLinear as TrainLinear
        for dtype in (torch.float16, torch.float32):
            for k, n in ((4096, 11008), (11008, 4096), (4096, 4096)):
                lin = TrainLinear(k, n, bias=False, w_bits=4, group_size=args.group, cherryq=True).to(dtype).cuda()
                lin.weight.data.normal_(0, 0.02)
                lin.register_cherry_indices(torch.randperm(k)[:lin.num_cherries])
                dst = torch.empty_like(lin.weight)
                wsrc = lin.weight.detach()

                def timed(fn, reps):
                    for _ in range(3):
                        fn()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(reps):
                        fn()
                    e1.record()
                    torch.cuda.synchronize()
                    return e0.elapsed_time(e1) / reps * 1e3

                us = timed(lambda: quant_cuda.fake_quant_cherryq(4, wsrc, lin.cherry_indices, args.group, out=dst), 50)
                lin._fused_fake_quant = lambda weight: False
                us_torch = timed(lambda: lin._adjust_weight(wsrc, ste=False), 5)
                ab = 2.0 * k * n * wsrc.element_size()
                print(f"fake-quant {str(dtype)[6:]:8s} {k:5d}->{n:5d}: {us:7.2f} us  {ab / us / 1e3:7.1f} GB/s "
                      f"({ab / us / 1e3 / HBM_PEAK_GBS * 100:4.1f}% of 8 TB/s; one read + one write of the weight)  "
                      f"torch operations {us_torch:8.1f} us", file=sys.stderr, flush=True)
                del lin, dst, wsrc
                torch.cuda.empty_cache()
        unpack_table(args.group)
        for name, (bits, k, n) in WORKLOADS.items():
            ab = algorithmic_bytes(bits, k, n, 1, args.group)
            line = f"{name:24s} {bits}-bit {k:5d}->{n:5d}:"
            for path in ("reference", "prepacked"):
                if path == "prepacked" and not quant_cuda.prepack_supported(bits, 1, k, n, -(-k // 256) // 8 * 8, args.group):
                    line += "  prepacked: shape not taken"
                    continue
                r = time_gpu(bits, k, n, args.group, max(200, args.steps // 4), args.warmup, use_graph=not args.no_graph,
                             path=path)
                line += (f"  {path} {r['us']:6.2f} us {ab / r['us'] / 1e3:6.0f} GB/s "
                         f"{ab / r['us'] / 1e3 / HBM_PEAK_GBS * 100:4.1f}%")
                del r
                torch.cuda.empty_cache()
            print(line, file=sys.stderr, flush=True)

    def kernel_name(bits, batch, path, k_in=0, n_out=0):
        if path == "prepacked":
            if batch == 1:
                import quant_cuda
                base_name = quant_cuda.prepacked_kernel_name(bits, k_in, n_out, -(-k_in // 256) // 8 * 8) if k_in and n_out else ""
                return f"{base_name or 'cq::stream_cu_kernel'}<{bits}>"
            import quant_cuda
            return f"{quant_cuda.prepacked_kernel_name(bits, k_in, n_out, -(-k_in // 256) // 8 * 8, rows=batch)} <{bits}-bit>"
        if batch == 1:
            return f"cq::matvec_kernel<{bits}>"
        if batch <= 4:
            return f"cq::matvec_kernel<{bits}, rows {2 if batch == 2 else 4}>"
        if batch <= 16:
            return f"cq::batch_prep_kernel<{bits}> + cq::batch_kernel<{bits}>"
        return f"cq::gemm_prep_kernel<{bits}> + cq::gemm_kernel<{bits}, {32 if batch <= 32 else 64 if batch <= 64 else 128}>"

    side_steps = min(args.steps, 500)

    def batch_record(name, batch, mfma=None):
        """A small-batch call (2..16 rows) on the path a loader gets for the layer: whole-call device time
        (preparation launch included), bytes, flops; `mfma`: matrix-core busy share from a recorded PMC run."""
        b_, k_, n_ = WORKLOADS[name]
        r = time_gpu(b_, k_, n_, args.group, side_steps, min(args.warmup, 50), batch=batch, use_graph=not args.no_graph)
        ab_ = algorithmic_bytes(b_, k_, n_, batch, args.group)
        fl = 2.0 * batch * k_ * n_
        rec = {"workload": name, "batch": batch, "us": round(r["us"], 3), "path": r["path"],
               "kernel": kernel_name(b_, batch, r["path"], k_, n_), "algorithmic_bytes_per_call": ab_,
               "achieved": round(ab_ / r["us"] / 1e3, 1), "unit": "GB/s", "frac": round(ab_ / r["us"] / 1e3 / HBM_PEAK_GBS, 4),
               "tflops": round(fl / r["us"] / 1e6, 1), "frac_of_fp16_mfma_peak": round(fl / r["us"] / 1e6 / 2500, 4)}
        if mfma:
            rec["mfma_busy"] = mfma
        del r
        torch.cuda.empty_cache()
        return rec

    def side_record(name, with_cpu=False):
        """One more layer in the same JSON line: both paths' device time, achieved bandwidth of the faster."""
        b_, k_, n_ = WORKLOADS[name]
        ab_ = algorithmic_bytes(b_, k_, n_, 1, args.group)
        rec = {"workload": name, "w_bits": b_, "in_features": k_, "out_features": n_, "algorithmic_bytes_per_launch": ab_}
        best = None
        for path in ("reference", "prepacked"):
            import quant_cuda
            if path == "prepacked" and not quant_cuda.prepack_supported(b_, 1, k_, n_, -(-k_ // 256) // 8 * 8, args.group):
                continue
            r = time_gpu(b_, k_, n_, args.group, side_steps, min(args.warmup, 50), use_graph=not args.no_graph, path=path)
            rec[f"{path}_us"] = round(r["us"], 3)
            if best is None or r["us"] < best[0]:
                best = (r["us"], path)
            if with_cpu and path == "reference" and not args.no_cpu:
                rec["cpu_baseline"] = cpu_baseline(b_, k_, n_, args.group, r["base"], r["x"].cpu().numpy(), seconds=4.0)
            del r
            torch.cuda.empty_cache()
        rec.update({"us": round(best[0], 3), "path": best[1], "kernel": kernel_name(b_, 1, best[1], k_, n_),
                    "achieved": round(ab_ / best[0] / 1e3, 1), "unit": "GB/s", "peak": HBM_PEAK_GBS,
                    "frac": round(ab_ / best[0] / 1e3 / HBM_PEAK_GBS, 4)})
        return rec

    bits, k, n = WORKLOADS[args.workload]
    main_run = time_gpu(bits, k, n, args.group, args.steps, args.warmup, batch=args.batch, use_graph=not args.no_graph)
    us, path = main_run["us"], main_run["path"]
    ab = algorithmic_bytes(bits, k, n, args.batch, args.group)
    gbs = ab / us / 1e3
    x_host = main_run["x"].cpu().numpy()
    base = main_run["base"]
    traffic = MEASURED_TRAFFIC.get((args.workload, args.batch, path))
    result = {
        "metric": "us_per_matvec", "value": round(us, 3), "unit": "us", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us / 1e3, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16xu%d->f32" % bits,
        "data": "synthetic",
        "config": {"workload": args.workload, "w_bits": bits, "in_features": k, "out_features": n,
                   "group_size": args.group, "batch": args.batch, "cherries": -(-k // 256) // 8 * 8,
                   "weight_copies_rotated": len(main_run["copies"]),
                   "path": path + (" (weight stream repacked once at load time from the reference buffers)"
                                   if path == "prepacked" else " (kernels that read the checkpoint layout)"),
                   "launch": "eager" if args.no_graph else "hip_graph_replay",
                   "replays": None if args.no_graph else _replays(args.steps),
                   "timing": ("one HIP graph of steps x replays launches; median over %d timed graph launches of "
                              "(HIP-event time / launches)" % TIMED_REPLAYS),
                   "eager_host_wall_us_per_call": round(main_run["wall_us"], 2)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": traffic,
                     "traffic_source": ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this workload and kernel, recorded in "
                                        "bench.py (profiles/); not re-measured in this run") if traffic else
                                       "not measured for this workload / kernel",
                     "algorithmic_bytes_per_launch": ab,
                     "kernel": kernel_name(bits, args.batch, path, k, n)},
    }
    if main_run["resident_us"] is not None:
        ru = main_run["resident_us"]
        result["roofline"]["cache_resident"] = {"us": round(ru, 3), "gbs": round(ab / ru / 1e3, 1),
                                                "note": "one weight copy replayed: served by the Infinity Cache, not HBM"}
    del main_run
    torch.cuda.empty_cache()
    if args.batch == 1 and not args.no_graph:
        if path == "prepacked":
            other = time_gpu(bits, k, n, args.group, args.steps, args.warmup, use_graph=True, path="reference")
            result["config"]["reference_layout_us"] = round(other["us"], 3)
            result["config"]["reference_layout_kernel"] = kernel_name(bits, 1, "reference")
            del other
            torch.cuda.empty_cache()
        result["roofline"]["reference"] = roofline_reference(ab, args.steps)
        if not args.no_decode:
            result["decode"] = decode_benchmark()
        if args.workload == "llama7b_gate_up_w4":
            # the other half of the headline metric (3-bit, same layer) and config 0 (4096 -> 4096,
            # 4-bit, with the reference's CPU path on that layer)
            result["roofline_w3"] = side_record("llama7b_gate_up_w3")
            result["config0"] = side_record("llama7b_attn_w4", with_cpu=True)
            # the rest of the configurations: the down projection of config 1, the LLaMA-13B shapes in
            # 3 bits at batch 1 / 4 / 8 (config 3), the LLaMA-70B shapes in 4 bits at batch 1 / 16 (config 4)
            result["config1_down"] = [side_record("llama7b_down_w4"), side_record("llama7b_down_w3")]
            result["config3"] = {"batch1": [side_record(w) for w in ("llama13b_attn_w3", "llama13b_gate_up_w3", "llama13b_down_w3")],
                                 "batched": [batch_record(w, b, MFMA_BUSY.get((w, b))) for w in ("llama13b_attn_w3", "llama13b_gate_up_w3") for b in (4, 8)]}
            result["config4"] = {"batch1": [side_record(w) for w in ("llama70b_attn_w4", "llama70b_kv_w4", "llama70b_gate_up_w4",
                                                                     "llama70b_down_w4")],
                                 "batch16": [batch_record("llama70b_gate_up_w4", 16, MFMA_BUSY.get("llama70b_gate_up_w4")),
                                             batch_record("llama70b_down_w4", 16, MFMA_BUSY.get("llama70b_down_w4"))]}
    if not args.no_decode and "decode" not in result:
        result["decode"] = decode_benchmark()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(bits, k, n, args.group, base, x_host)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
