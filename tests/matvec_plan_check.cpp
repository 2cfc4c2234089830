// Host-side check of the split-K geometry of the batch-1 .. 4-row streaming kernel over the
// checkpoint layout (cq::matvec_geometry / cq::matvec_supported), over a sweep of shapes that
// includes very long rows of small layers: whenever a shape is reported as supported, the
// geometry the launch will use must keep the workgroups per column tile within the 8-bit arrival
// counter of the split-K accumulator word (255), cover every unit, and a shape whose geometry
// cannot do so must be reported as not supported.  Built and run by test_matvec_plan.py with the
// host compiler; prints the offending shapes and returns 1.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdio>

#include "../mixed-precision-cuda-kernel_amd/csrc/cq_kernels.h"

int main() {
    const int Ks[] = {64,    256,   1024,  4096,  4104,  8192,  11008, 16384,  28672,  32768,
                      40960, 65280, 65288, 65536, 66000, 98304, 130560, 130568, 131072, 200000};
    const int Ns[] = {8, 16, 64, 256, 1024, 4096, 11008, 28672, 128256};
    long bad = 0, count = 0, refused = 0;
    for (int bits = 3; bits <= 4; bits++)
        for (int rows = 1; rows <= 4; rows++)
            for (int K : Ks)
                for (int N : Ns)
                    for (int cf = 0; cf < 2; cf++) {
                        const int C = cf == 0 || K > 32768 ? 0 : (K + 255) / 256 / 8 * 8;
                        if (cf == 1 && C == 0) continue;
                        if (K - C <= 0) continue;
                        count++;
                        const cq::MatvecGeometry g = cq::matvec_geometry(bits, K, N, C, rows);
                        const bool sup = cq::matvec_supported(bits, rows, K, N, C, 128);
                        const int unit = 4 * g.kpl;
                        const long units = (long)(K - C + unit - 1) / unit + (C + 31) / 32;
                        bool ok = (g.kpl == 16 || g.kpl == 32) && (g.nw == 1 || g.nw == 2 || g.nw == 4) && g.splits >= 1 &&
                                  (long)g.splits * g.nw >= units && (long)(g.splits - 1) * g.nw < units;
                        if (sup && g.splits > 255) ok = false;       // the counter would wrap: silent wrong sums
                        const long long wbytes = (long long)(K - C) / 8 * 4 * N;
                        if (!sup && g.splits <= 255 && wbytes < 0x7fff0000ll) ok = false;  // refused without a reason
                        if (!sup) refused++;
                        if (!ok) {
                            bad++;
                            std::printf("bad: bits %d rows %d K %d N %d C %d -> unit %d waves %d splits %d supported %d\n", bits,
                                        rows, K, N, C, unit, g.nw, g.splits, (int)sup);
                        }
                    }
    std::printf("%ld shapes checked, %ld refused, %ld bad\n", count, refused, bad);
    return bad ? 1 : 0;
}
