// GEMM core, matrix-core strategy: bit planes are re-assembled to int8 in registers and fed to
// v_mfma_i32_16x16x64_i8 / v_mfma_i32_32x32x32_i8 (gfx950).
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271 and :485-580) for one (x_bits, w_bits) pair per
// translation unit: compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>.
//
// Work split.  A workgroup owns a BM x BN tile of D.  Its WM x WN x WK waves tile M and N and
// interleave the K steps among the WK waves of a tile (partial sums meet in LDS).  A wave owns
// TM x TN MFMA tiles of MI x MI outputs.
//
// Operand mapping.  The MFMA wants from lane l the row (l % MI) of A (resp. column of B) and
// the K group (l / MI).  Lane l therefore loads, for each of its rows and each plane, the four
// consecutive plane words [step*STEPW + 4*(l/MI), +4) with one 16-byte load straight from the
// reference layout, expands each word (32 K elements) to 32 int8 with a 3-stage bit-matrix
// transpose, and issues two MFMAs per word.  Activation and weight words are expanded by the
// same routine, so their K elements line up whatever the bit widths are.
//
// Integer exactness.
//   signed    planes sit at the top of the byte, the MFMA sums x*2^(8-Q) * w*2^(8-P); the
//             epilogue shifts right by 16-Q-P.  |sum| <= K * 2^14, so K < 2^17 is required.
//   unsigned  up to 7 bits fit an int8 as they are.  An 8-bit unsigned operand is fed as
//             value - 128 (bit 7 flipped) and the epilogue adds 128 * (row sum of the other
//             operand), minus 2^14 * K when both are 8-bit.  Row sums are popcounts of the
//             plane words the lane already holds.
#include "abq_kernels.h"

#ifndef ABQ_Q
#error "compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>"
#endif

namespace abq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

template <int MI> struct Mfma;
template <> struct Mfma<16> {
    typedef v4i acc_t;
    static constexpr int kAcc = 4;
    static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c)
    {
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
    }
    // row of the MI x MI tile held in accumulator element e by a lane of group g
    static __device__ __forceinline__ int row(int e, int g) { return 4 * g + e; }
};
template <> struct Mfma<32> {
    typedef v16i acc_t;
    static constexpr int kAcc = 16;
    static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c)
    {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int e, int g) { return 8 * (e / 4) + 4 * g + (e % 4); }
};

__device__ __forceinline__ uint32_t comp(const uint4 &v, int i)
{
    return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

template <int BITS>
__device__ __forceinline__ void load_planes(uint4 (&dst)[BITS], const uint32_t *row_ptr,
                                            size_t plane_stride, int word, bool valid)
{
#pragma unroll
    for (int b = 0; b < BITS; ++b) {
        if (valid)
            dst[b] = *reinterpret_cast<const uint4 *>(row_ptr + b * plane_stride + word);
        else
            dst[b] = make_uint4(0u, 0u, 0u, 0u);
    }
}

template <int Q, int P, bool SIGNED, int MI, int TM, int TN, int WM, int WN, int WK>
__global__ __launch_bounds__(64 * WM * WN * WK) void gemm_mfma_direct(const GemmArgs a)
{
    typedef Mfma<MI> MF;
    typedef typename MF::acc_t acc_t;
    constexpr int G = 64 / MI;      // K groups (lane / MI)
    constexpr int STEPW = 4 * G;    // plane words per row consumed per step
    constexpr int kAcc = MF::kAcc;
    constexpr Int8Mode XMODE = Int8ModeOf<Q, SIGNED>::value;
    constexpr Int8Mode WMODE = Int8ModeOf<P, SIGNED>::value;
    constexpr bool X_IS_U8 = XMODE == kFlip;
    constexpr bool W_IS_U8 = WMODE == kFlip;
    constexpr bool NEED_SX = W_IS_U8; // 128 * sum_k x[m,k] enters when W was fed as w - 128
    constexpr bool NEED_SW = X_IS_U8;

    const int lane = threadIdx.x & 63;
    const int wid = threadIdx.x >> 6;
    const int wk = wid % WK;
    const int wn = (wid / WK) % WN;
    const int wm = wid / (WK * WN);
    const int r = lane % MI;
    const int g = lane / MI;

    const int M = a.M, N = a.N, KW = a.KW;
    const int m_base = blockIdx.y * (MI * TM * WM) + wm * (MI * TM);
    const int n_base = blockIdx.x * (MI * TN * WN) + wn * (MI * TN);
    const int nsteps = (KW + STEPW - 1) / STEPW;
    const size_t xplane = (size_t)M * KW;
    const size_t wplane = (size_t)N * KW;

    // Rows past the edge are clamped for loading; their results are dropped at the store.
    const uint32_t *xrow[TM];
    const uint32_t *wrow[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t)
        xrow[t] = a.X + (size_t)min(m_base + t * MI + r, M - 1) * KW;
#pragma unroll
    for (int t = 0; t < TN; ++t)
        wrow[t] = a.W + (size_t)min(n_base + t * MI + r, N - 1) * KW;

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < kAcc; ++e)
                acc[i][j][e] = 0;
    int sx[TM], sw[TN]; // partial row sums of the unsigned values (8-bit unsigned operands only)
#pragma unroll
    for (int t = 0; t < TM; ++t)
        sx[t] = 0;
#pragma unroll
    for (int t = 0; t < TN; ++t)
        sw[t] = 0;

    uint4 cx[TM][Q], cw[TN][P]; // plane words of the step being computed
    uint4 nx[TM][Q], nw[TN][P]; // and of the next one (register double buffer)

    {
        const int word = wk * STEPW + 4 * g;
        const bool valid = word < KW;
#pragma unroll
        for (int t = 0; t < TM; ++t)
            load_planes<Q>(cx[t], xrow[t], xplane, word, valid);
#pragma unroll
        for (int t = 0; t < TN; ++t)
            load_planes<P>(cw[t], wrow[t], wplane, word, valid);
    }

    for (int s = wk; s < nsteps; s += WK) {
        {
            const int word = (s + WK) * STEPW + 4 * g;
            const bool valid = word < KW; // false past the last step: no memory access
#pragma unroll
            for (int t = 0; t < TM; ++t)
                load_planes<Q>(nx[t], xrow[t], xplane, word, valid);
#pragma unroll
            for (int t = 0; t < TN; ++t)
                load_planes<P>(nw[t], wrow[t], wplane, word, valid);
        }

#pragma unroll
        for (int ws = 0; ws < 4; ++ws) {
            uint32_t aop[TM][8], bop[TN][8];
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                uint32_t w[Q];
#pragma unroll
                for (int b = 0; b < Q; ++b)
                    w[b] = comp(cx[t][b], ws);
                if (NEED_SX)
                    sx[t] += planes_value_sum<Q>(w);
                planes_to_int8<Q, XMODE>(w, aop[t]);
            }
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                uint32_t w[P];
#pragma unroll
                for (int b = 0; b < P; ++b)
                    w[b] = comp(cw[t][b], ws);
                if (NEED_SW)
                    sw[t] += planes_value_sum<P>(w);
                planes_to_int8<P, WMODE>(w, bop[t]);
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const v4i av = { (int)aop[i][4 * h], (int)aop[i][4 * h + 1],
                                     (int)aop[i][4 * h + 2], (int)aop[i][4 * h + 3] };
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        const v4i bv = { (int)bop[j][4 * h], (int)bop[j][4 * h + 1],
                                         (int)bop[j][4 * h + 2], (int)bop[j][4 * h + 3] };
                        acc[i][j] = MF::run(av, bv, acc[i][j]);
                    }
                }
            }
        }

#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int b = 0; b < Q; ++b)
                cx[t][b] = nx[t][b];
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int b = 0; b < P; ++b)
                cw[t][b] = nw[t][b];
    }

    // Row sums: add up the K groups of the wave (lanes r, r+MI, ...).
    if (NEED_SX) {
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int off = MI; off < 64; off <<= 1)
                sx[t] += __shfl_xor(sx[t], off, 64);
    }
    if (NEED_SW) {
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int off = MI; off < 64; off <<= 1)
                sw[t] += __shfl_xor(sw[t], off, 64);
    }

    // Waves that split K meet in LDS; the wk == 0 wave of each tile finishes.
    if (WK > 1) {
        constexpr int PER_WAVE = (TM * TN * kAcc + TM + TN) * 64;
        __shared__ int red[WM * WN * (WK > 1 ? WK - 1 : 1) * PER_WAVE];
        if (wk != 0) {
            int *dst = red + ((wm * WN + wn) * (WK - 1) + (wk - 1)) * PER_WAVE + lane;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < kAcc; ++e)
                        dst[((i * TN + j) * kAcc + e) * 64] = acc[i][j][e];
#pragma unroll
            for (int t = 0; t < TM; ++t)
                dst[(TM * TN * kAcc + t) * 64] = sx[t];
#pragma unroll
            for (int t = 0; t < TN; ++t)
                dst[(TM * TN * kAcc + TM + t) * 64] = sw[t];
        }
        __syncthreads();
        if (wk != 0)
            return;
        for (int k2 = 0; k2 < WK - 1; ++k2) {
            const int *src = red + ((wm * WN + wn) * (WK - 1) + k2) * PER_WAVE + lane;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < kAcc; ++e)
                        acc[i][j][e] += src[((i * TN + j) * kAcc + e) * 64];
#pragma unroll
            for (int t = 0; t < TM; ++t)
                sx[t] += src[(TM * TN * kAcc + t) * 64];
#pragma unroll
            for (int t = 0; t < TN; ++t)
                sw[t] += src[(TM * TN * kAcc + TM + t) * 64];
        }
    }

    const int k_fed = nsteps * STEPW * 32; // K elements fed to the MFMAs including zero fill
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n_base + j * MI + r;
#pragma unroll
            for (int e = 0; e < kAcc; ++e) {
                const int il = MF::row(e, g);
                const int m = m_base + i * MI + il;
                unsigned v = (unsigned)acc[i][j][e];
                if (SIGNED) {
                    v = (unsigned)((int)v >> (16 - Q - P));
                } else {
                    if (NEED_SX)
                        v += 128u * (unsigned)__shfl(sx[i], il, 64);
                    if (NEED_SW)
                        v += 128u * (unsigned)sw[j];
                    if (NEED_SX && NEED_SW)
                        v -= 16384u * (unsigned)k_fed;
                }
                if (m < M && n < N)
                    store_result(a, m, n, (int)v);
            }
        }
    }
}

template <int Q, int P, bool SIGNED, int MI, int TM, int TN, int WM, int WN, int WK>
static hipError_t launch_mfma_direct(const GemmArgs &a, hipStream_t stream)
{
    const dim3 grid((a.N + MI * TN * WN - 1) / (MI * TN * WN), (a.M + MI * TM * WM - 1) / (MI * TM * WM));
    const dim3 block(64 * WM * WN * WK);
    hipLaunchKernelGGL((gemm_mfma_direct<Q, P, SIGNED, MI, TM, TN, WM, WN, WK>), grid, block, 0,
                       stream, a);
    return hipGetLastError();
}

// The native tile space of this strategy, V(MI, TM, TN, WM, WN, WK), is the list the tile
// generator emits (engine/gen_kernel.cpp, --format variants).
#define ABQ_MFMA_VARIANTS(V) \
    V(16, 1, 1, 1, 1, 4) \
    V(16, 1, 1, 1, 1, 8) \
    V(16, 1, 1, 1, 2, 2) \
    V(16, 1, 1, 1, 2, 4) \
    V(16, 1, 2, 1, 1, 4) \
    V(16, 1, 2, 1, 1, 8) \
    V(16, 1, 2, 1, 2, 2) \
    V(16, 1, 2, 1, 2, 4) \
    V(32, 1, 1, 2, 2, 1) \
    V(32, 1, 2, 2, 2, 1) \
    V(32, 2, 2, 2, 2, 1)

#define ABQ_ENTRY(S, MI, TM, TN, WM, WN, WK) \
    { MI, TM, TN, WM, WN, WK, 2, &launch_mfma_direct<ABQ_Q, ABQ_P, S, MI, TM, TN, WM, WN, WK> },
#define ABQ_ENTRY_T(MI, TM, TN, WM, WN, WK) ABQ_ENTRY(true, MI, TM, TN, WM, WN, WK)
#define ABQ_ENTRY_F(MI, TM, TN, WM, WN, WK) ABQ_ENTRY(false, MI, TM, TN, WM, WN, WK)

static const KernelEntry kSigned[] = { ABQ_MFMA_VARIANTS(ABQ_ENTRY_T) };
static const KernelEntry kUnsigned[] = { ABQ_MFMA_VARIANTS(ABQ_ENTRY_F) };

#define ABQ_CAT_(a, b, c, d) a##b##c##d
#define ABQ_CAT(a, b, c, d) ABQ_CAT_(a, b, c, d)

// abq_mfma_register_<Q>_<P>: fills two tables (signed, unsigned).
void ABQ_CAT(abq_mfma_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSigned, (int)(sizeof(kSigned) / sizeof(kSigned[0])) };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsigned, (int)(sizeof(kUnsigned) / sizeof(kUnsigned[0])) };
}

} // namespace abq
