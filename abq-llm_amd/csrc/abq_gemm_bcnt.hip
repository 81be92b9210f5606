// GEMM core, VALU strategy: AND + popcount on the packed planes, K along the lanes, wavefront
// reduction.  Meant for decode-sized M (one or two activation rows): every weight word is read
// exactly once with 16-byte loads straight from the reference layout and never expanded.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for one (x_bits, w_bits) pair per
// translation unit: compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>.
//
// Work split.  LPR = 2^lpr_log2 lanes share one weight row, so a wave covers 64/LPR rows per
// pass; lane c of a row handles the 16-byte units c, c+LPR, ... of that row (a unit is four
// plane words = 128 K elements).  Per unit and per activation row a lane does, for each of the
// Q*P plane pairs, 4 v_and + 4 v_bcnt (chained through the accumulate operand) and one
// multiply-add by +/-2^(i+j); the LPR partial sums meet through cross-lane shuffles.
// The activation words come from global memory on every pass; they are a few KiB and stay in
// the vector L1.
#include "abq_kernels.h"

#ifndef ABQ_Q
#error "compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>"
#endif

namespace abq {

__device__ __forceinline__ int popc4(const uint4 &x, const uint4 &w)
{
    return __builtin_popcount(x.x & w.x) + __builtin_popcount(x.y & w.y) +
           __builtin_popcount(x.z & w.z) + __builtin_popcount(x.w & w.w);
}

template <int Q, int P, bool SIGNED, int MT>
__global__ __launch_bounds__(256) void gemm_bcnt(const GemmArgs a)
{
    const int lane = threadIdx.x & 63;
    const int wid = threadIdx.x >> 6;
    const int lpr_log2 = a.lpr_log2;
    const int LPR = 1 << lpr_log2;
    const int RPP = 64 >> lpr_log2; // weight rows per wave pass
    const int M = a.M, N = a.N, KW = a.KW;
    const int units = KW >> 2;
    const int npass = (N + RPP - 1) / RPP;
    const int m0 = blockIdx.y * MT;
    const size_t xplane = (size_t)M * KW;
    const size_t wplane = (size_t)N * KW;
    const int lir = lane & (LPR - 1);

    const uint32_t *xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
        xrow[t] = a.X + (size_t)min(m0 + t, M - 1) * KW;

    for (int pass = blockIdx.x * 4 + wid; pass < npass; pass += gridDim.x * 4) {
        const int row = pass * RPP + (lane >> lpr_log2);
        const uint32_t *wrow = a.W + (size_t)min(row, N - 1) * KW;
        int acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t)
            acc[t] = 0;

        for (int u = lir; u < units; u += LPR) {
            uint4 w[P];
#pragma unroll
            for (int j = 0; j < P; ++j)
                w[j] = *reinterpret_cast<const uint4 *>(wrow + j * wplane + 4 * u);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
#pragma unroll
                for (int i = 0; i < Q; ++i) {
                    const uint4 x = *reinterpret_cast<const uint4 *>(xrow[t] + i * xplane + 4 * u);
#pragma unroll
                    for (int j = 0; j < P; ++j)
                        acc[t] += popc4(x, w[j]) * plane_pair_weight(i, j, Q, P, SIGNED);
                }
            }
        }

#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                if (off < LPR) // uniform over the wave
                    acc[t] += __shfl_xor(acc[t], off, 64);
            }
        }
        if (lir == 0 && row < N) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
                if (m0 + t < M)
                    store_result(a, m0 + t, row, acc[t]);
        }
    }
}

template <int Q, int P, bool SIGNED, int MT>
static hipError_t launch_bcnt(const GemmArgs &a, hipStream_t stream)
{
    const int rpp = 64 >> a.lpr_log2;
    const int npass = (a.N + rpp - 1) / rpp;
    int gx = (npass + 3) / 4;
    if (gx > 65536)
        gx = 65536; // the kernel strides over the passes
    const dim3 grid(gx, (a.M + MT - 1) / MT);
    hipLaunchKernelGGL((gemm_bcnt<Q, P, SIGNED, MT>), grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

// Native tile space of this strategy: activation rows per pass.
#define ABQ_BCNT_VARIANTS(V) V(1) V(2) V(4)

#define ABQ_ENTRY_T(MT) { 1, MT, 1, 1, 4, 1, 1, &launch_bcnt<ABQ_Q, ABQ_P, true, MT> },
#define ABQ_ENTRY_F(MT) { 1, MT, 1, 1, 4, 1, 1, &launch_bcnt<ABQ_Q, ABQ_P, false, MT> },

static const KernelEntry kSigned[] = { ABQ_BCNT_VARIANTS(ABQ_ENTRY_T) };
static const KernelEntry kUnsigned[] = { ABQ_BCNT_VARIANTS(ABQ_ENTRY_F) };

#define ABQ_CAT_(a, b, c, d) a##b##c##d
#define ABQ_CAT(a, b, c, d) ABQ_CAT_(a, b, c, d)

void ABQ_CAT(abq_bcnt_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSigned, (int)(sizeof(kSigned) / sizeof(kSigned[0])) };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsigned, (int)(sizeof(kUnsigned) / sizeof(kUnsigned[0])) };
}

} // namespace abq
