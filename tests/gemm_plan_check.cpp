// Host-side check of the K-split plan of the prompt-sized path (cq::gemm_plan), over a sweep of
// shapes: every plan must cover all K steps exactly once with at least one split, keep the step
// count per split in the form the kernel's unrolled loop takes, size the partial tiles for the
// splits it launches, and split only when all workgroups are resident at once.  Built and run
// by test_gemm_plan.py with the host compiler; prints the offending plans and returns 1.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdio>

#include "../mixed-precision-cuda-kernel_amd/csrc/cq_kernels.h"

int main() {
    const int Ms[] = {17, 24, 40, 63, 64, 65, 100, 128, 129, 256, 511, 1000, 2048, 5000};
    const int Ks[] = {64, 256, 512, 1024, 4096, 4104, 5120, 8192, 11008, 13824, 28672};
    const int Ns[] = {8, 64, 264, 1024, 4096, 11008, 28672, 98304, 98312, 128256, 200000};
    long bad = 0, count = 0;
    for (int M : Ms)
        for (int K : Ks)
            for (int N : Ns)
                for (int cf = 0; cf < 3; cf++) {
                    const int C = cf == 0 ? 0 : cf == 1 ? (K + 255) / 256 / 8 * 8 : K / 8 / 8 * 8;
                    if (K - C <= 0) continue;
                    const cq::GemmPlan p = cq::gemm_plan(M, K, N, C);
                    count++;
                    const int tm = p.tm;
                    const long wgs = (long)p.mtiles * p.ntiles * p.splits;
                    const bool ok =
                        (tm == 32 || tm == 64 || tm == 128) && p.splits >= 1 && p.splits <= 16 && p.steps_per_split >= 1 &&
                        (long)p.splits * p.steps_per_split >= p.steps_total &&
                        (long)(p.splits - 1) * p.steps_per_split < p.steps_total &&
                        (p.splits == 1 || (p.steps_per_split - 2) % 6 == 0) && p.mtiles * tm >= M &&
                        (p.mtiles - 1) * tm < M && p.Mp == p.mtiles * tm && p.Kp == p.steps_total * 64 &&
                        p.steps_total * 64 >= K && p.ntiles * 128 >= N && (p.ntiles - 1) * 128 < N &&
                        p.partial_bytes ==
                            (p.splits > 1 ? (size_t)p.splits * p.mtiles * p.ntiles * tm * 128 * sizeof(float) : 0) &&
                        p.a_bytes >= (size_t)p.Mp * p.Kp * 2 && p.scratch_bytes >= p.a_bytes + p.partial_bytes &&
                        (p.splits == 1 || wgs <= 1024);
                    if (!ok) {
                        bad++;
                        std::printf("bad plan: M %d K %d N %d C %d -> tile rows %d tiles %d x %d steps %d splits %d x %d\n",
                                    M, K, N, C, p.tm, p.mtiles, p.ntiles, p.steps_total, p.splits,
                                    p.steps_per_split);
                    }
                }
    std::printf("%ld plans checked, %ld bad\n", count, bad);
    return bad ? 1 : 0;
}
