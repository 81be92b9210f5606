// GEMM core, fallback: the popcount formulation with run-time bit widths (1..16 each).
// Serves bit combinations without a specialised instantiation, such as the W1A1 / W1A4 /
// W1A8 / W1A16 / W2A16 samples of the reference library (engine/mma_any/aq_bmma_library.cu:18-66).
// One wave per weight row, lanes along K, same sum as engine/test_any_mma.cu:58-84.
#include "abq_kernels.h"

namespace abq {

__global__ __launch_bounds__(256) void gemm_bcnt_generic(const GemmArgs a, int x_bits, int w_bits,
                                                          int is_signed)
{
    const int lane = threadIdx.x & 63;
    const int wid = threadIdx.x >> 6;
    const int M = a.M, N = a.N, KW = a.KW;
    const size_t xplane = (size_t)M * KW;
    const size_t wplane = (size_t)N * KW;
    const int m = blockIdx.y;

    for (int n = blockIdx.x * 4 + wid; n < N; n += gridDim.x * 4) {
        int acc = 0;
        for (int i = 0; i < x_bits; ++i) {
            const uint32_t *xr = a.X + i * xplane + (size_t)m * KW;
            for (int j = 0; j < w_bits; ++j) {
                const uint32_t *wr = a.W + j * wplane + (size_t)n * KW;
                int cnt = 0;
                for (int kw = lane; kw < KW; kw += 64)
                    cnt += __builtin_popcount(xr[kw] & wr[kw]);
                acc += cnt * plane_pair_weight(i, j, x_bits, w_bits, is_signed != 0);
            }
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1)
            acc += __shfl_xor(acc, off, 64);
        if (lane == 0)
            store_result(a, m, n, acc);
    }
}

hipError_t launch_bcnt_generic(const GemmArgs &a, int x_bits, int w_bits, int is_signed,
                               hipStream_t stream)
{
    int gx = (a.N + 3) / 4;
    if (gx > 65536)
        gx = 65536;
    hipLaunchKernelGGL(gemm_bcnt_generic, dim3(gx, a.M), dim3(256), 0, stream, a, x_bits, w_bits,
                       is_signed);
    return hipGetLastError();
}

} // namespace abq
