// GEMM core for prefill-sized M: matrix-core strategy, LDS-staged, operands in the K-tiled
// plane layout.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for one (x_bits, w_bits) pair per
// translation unit: compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>.
//
// Why a second layout.  In the reference layout a K tile of 128 elements is 16 bytes per
// (row, plane) and rows are K/8 bytes apart, so a workgroup tile touches one 128-byte cache line
// per 16 useful bytes; with hundreds of rows per tile the vector L1 fill rate, not the matrix
// cores, bounds the kernel.  The K-tiled layout keeps the same bits in the order
//     tiled[kt][row][plane][4 words],  kt = K tile of 128 elements,
// so the rows of a tile are contiguous (bits*16 bytes each) and every line is used in full.
// Weights are converted once (they are static), activations once per call; see
// relayout_planes_kernel below.
//
// Work split.  256 threads = 2 x 2 waves; a wave owns TM x TN MFMA tiles of 32 x 32, the
// workgroup tile is (64*TM) x (64*TN), the K tile 128.  Per K tile each thread expands the
// plane words of at most one activation row and one weight row to int8 (abq_bits.h) and
// writes them to LDS, so every row is expanded once per workgroup; the waves read their MFMA
// operands with ds_read_b128 (row stride 144 bytes: conflict free).  LDS is double buffered
// and the plane words of the next two K tiles are in flight in registers, so the expansion
// of tile i+1 and the loads of tile i+2 overlap the MFMAs of tile i; one barrier per K tile.
// Workgroups are numbered so that the 8 XCDs (workgroup id modulo 8) each work on a
// contiguous band of N with M fastest: a band's weight panels stay in that XCD's L2.
#include <type_traits>

#include "abq_kernels.h"

#ifndef ABQ_Q
#error "compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>"
#endif

namespace abq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTileK = 128;        // K elements per tile
constexpr int kLdsRow = 144;       // bytes per expanded row in LDS (128 + 16 padding)

template <int BITS>
__device__ __forceinline__ void load_tile_row(uint4 (&dst)[BITS], const uint32_t *tiled, int rows, int row, int kt)
{
    const uint4 *p = reinterpret_cast<const uint4 *>(tiled) + ((size_t)kt * rows + row) * BITS;
#pragma unroll
    for (int b = 0; b < BITS; ++b)
        dst[b] = p[b];
}

__device__ __forceinline__ uint32_t comp_t(const uint4 &v, int i)
{
    return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

// Expands the 4 word-sets of one row (128 K elements) and writes 128 int8 to LDS.
template <int BITS, Int8Mode MODE, bool SUM>
__device__ __forceinline__ void expand_row_to_lds(const uint4 (&raw)[BITS], unsigned char *lds_row, int &value_sum)
{
#pragma unroll
    for (int ws = 0; ws < 4; ++ws) {
        uint32_t w[BITS], o[8];
#pragma unroll
        for (int b = 0; b < BITS; ++b)
            w[b] = comp_t(raw[b], ws);
        if (SUM)
            value_sum += planes_value_sum<BITS>(w);
        planes_to_int8<BITS, MODE>(w, o);
        uint4 *dst = reinterpret_cast<uint4 *>(lds_row + ws * 32);
        dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
        dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
    }
}

template <int Q, int P, bool SIGNED, int TM, int TN>
__global__ __launch_bounds__(256) void gemm_mfma_tiled(const GemmArgs a, const uint32_t *xt, const uint32_t *wt,
                                                        int m_blocks, int n_blocks_per_xcd)
{
    constexpr int BM = 64 * TM, BN = 64 * TN;
    constexpr int UNITS = BM + BN;                 // rows expanded per K tile
    constexpr bool SPLIT = UNITS <= 256;           // each thread expands one row: A rows first, then B rows
    constexpr int NA = SPLIT ? 1 : (BM + 255) / 256; // else every thread expands NA rows of A and NB of B
    constexpr int NB = SPLIT ? 1 : (BN + 255) / 256;
    constexpr Int8Mode XMODE = Int8ModeOf<Q, SIGNED>::value;
    constexpr Int8Mode WMODE = Int8ModeOf<P, SIGNED>::value;
    constexpr bool NEED_SX = WMODE == kFlip; // see abq_gemm_mfma.hip
    constexpr bool NEED_SW = XMODE == kFlip;
    constexpr int BUF_BYTES = UNITS * kLdsRow;

    extern __shared__ __align__(16) unsigned char smem[];
    // [2][BM + BN][144] expanded rows, then row sums [BM + BN]
    int *rowsum = reinterpret_cast<int *>(smem + 2 * BUF_BYTES);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = tid >> 6;
    const int wm = wid >> 1, wn = wid & 1;
    const int r = lane & 31, g = lane >> 5;
    const int M = a.M, N = a.N;
    const int ktiles = a.K / kTileK;

    // workgroup -> tile: XCD x = id % 8 owns n blocks [x * npx, (x+1) * npx), M fastest
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int nb = xcd * n_blocks_per_xcd + slot / m_blocks;
    const int mb = slot % m_blocks;
    const int m0 = mb * BM, n0 = nb * BN;
    if (n0 >= N)
        return; // uniform over the workgroup, before any barrier

    // the rows this thread expands (fixed for the whole K loop; activity is uniform per wave)
    bool act_a[NA], act_b[NB];
    int la[NA], lb[NB];   // row within the tile
    int ga[NA], gb[NB];   // row in the operand (clamped at the edge, dropped at the store)
#pragma unroll
    for (int u = 0; u < NA; ++u) {
        la[u] = tid + u * 256;
        act_a[u] = la[u] < BM;
        ga[u] = min(m0 + la[u], M - 1);
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        lb[u] = SPLIT ? tid - BM : tid + u * 256;
        act_b[u] = lb[u] >= 0 && lb[u] < BN;
        gb[u] = min(n0 + max(lb[u], 0), N - 1);
    }

    uint4 rawx[2][NA][Q], raww[2][NB][P]; // plane words of the next two K tiles
    int sum_a[NA], sum_b[NB];
#pragma unroll
    for (int u = 0; u < NA; ++u)
        sum_a[u] = 0;
#pragma unroll
    for (int u = 0; u < NB; ++u)
        sum_b[u] = 0;

    // register slots are named at compile time (S0 / S1) so that the arrays stay in registers
    auto load_tile = [&](int kt, auto slot_c) __attribute__((always_inline)) {
        constexpr int slot_ = decltype(slot_c)::value;
        if (kt < ktiles) {
#pragma unroll
            for (int u = 0; u < NA; ++u)
                if (act_a[u])
                    load_tile_row<Q>(rawx[slot_][u], xt, M, ga[u], kt);
#pragma unroll
            for (int u = 0; u < NB; ++u)
                if (act_b[u])
                    load_tile_row<P>(raww[slot_][u], wt, N, gb[u], kt);
        }
    };
    auto expand_tile = [&](auto slot_c, int buf) __attribute__((always_inline)) {
        constexpr int slot_ = decltype(slot_c)::value;
        unsigned char *base = smem + buf * BUF_BYTES;
#pragma unroll
        for (int u = 0; u < NA; ++u)
            if (act_a[u])
                expand_row_to_lds<Q, XMODE, NEED_SX>(rawx[slot_][u], base + la[u] * kLdsRow, sum_a[u]);
#pragma unroll
        for (int u = 0; u < NB; ++u)
            if (act_b[u])
                expand_row_to_lds<P, WMODE, NEED_SW>(raww[slot_][u], base + (BM + lb[u]) * kLdsRow, sum_b[u]);
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[i][j][e] = 0;

    const std::integral_constant<int, 0> S0;
    const std::integral_constant<int, 1> S1;
    load_tile(0, S0);
    load_tile(1, S1);
    expand_tile(S0, 0);
    __syncthreads();

    const unsigned char *a_lane = smem + (wm * 32 * TM + r) * kLdsRow + g * 16;
    const unsigned char *b_lane = smem + (BM + wn * 32 * TN + r) * kLdsRow + g * 16;

    // One K tile: MFMAs on LDS buffer `buf` (tile kt), loads of tile kt+2 into the register slot
    // tile kt used, expansion of tile kt+1 (other register slot) into the other LDS buffer.
    auto k_tile = [&](int kt, auto cur_c, auto nxt_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(cur_c)::value;
        load_tile(kt + 2, cur_c);
        const unsigned char *ab = a_lane + buf * BUF_BYTES;
        const unsigned char *bb = b_lane + buf * BUF_BYTES;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            v4i av[TM], bv[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                av[i] = *reinterpret_cast<const v4i *>(ab + i * 32 * kLdsRow + ks * 32);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bv[j] = *reinterpret_cast<const v4i *>(bb + j * 32 * kLdsRow + ks * 32);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < ktiles)
            expand_tile(nxt_c, buf ^ 1);
        __syncthreads();
    };
    for (int kt = 0; kt < ktiles; kt += 2) {
        k_tile(kt, S0, S1);
        if (kt + 1 < ktiles)
            k_tile(kt + 1, S1, S0);
    }

    if (NEED_SX || NEED_SW) {
#pragma unroll
        for (int u = 0; u < NA; ++u)
            if (act_a[u])
                rowsum[la[u]] = sum_a[u];
#pragma unroll
        for (int u = 0; u < NB; ++u)
            if (act_b[u])
                rowsum[BM + lb[u]] = sum_b[u];
        __syncthreads();
    }

    const int k_fed = ktiles * kTileK;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int nl = wn * 32 * TN + j * 32 + r;
            const int n = n0 + nl;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int ml = wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4);
                const int m = m0 + ml;
                unsigned v = (unsigned)acc[i][j][e];
                if (SIGNED) {
                    v = (unsigned)((int)v >> (16 - Q - P));
                } else {
                    if (NEED_SX)
                        v += 128u * (unsigned)rowsum[ml];
                    if (NEED_SW)
                        v += 128u * (unsigned)rowsum[BM + nl];
                    if (NEED_SX && NEED_SW)
                        v -= 16384u * (unsigned)k_fed;
                }
                if (m < M && n < N)
                    store_result(a, m, n, (int)v);
            }
        }
    }
}

template <int Q, int P, bool SIGNED, int TM, int TN>
static hipError_t launch_mfma_tiled(const GemmArgs &a, hipStream_t stream)
{
    constexpr int BM = 64 * TM, BN = 64 * TN;
    const int m_blocks = (a.M + BM - 1) / BM, n_blocks = (a.N + BN - 1) / BN;
    const int npx = (n_blocks + 7) / 8;
    const size_t lds = 2 * (size_t)(BM + BN) * kLdsRow + (BM + BN) * sizeof(int);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_tiled<Q, P, SIGNED, TM, TN>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    const dim3 grid(8 * npx * m_blocks);
    hipLaunchKernelGGL((gemm_mfma_tiled<Q, P, SIGNED, TM, TN>), grid, dim3(256), lds, stream, a, a.X, a.W, m_blocks, npx);
    return hipGetLastError();
}

// Native tile space of this kernel: MFMA tiles per wave (TM, TN); nstage 4 marks the K-tiled
// operand layout.
#define ABQ_TILED_VARIANTS(V) V(4, 4) V(2, 4) V(2, 2) V(2, 1) V(1, 1)

#define ABQ_ENTRY_T(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, true, TM, TN> },
#define ABQ_ENTRY_F(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, false, TM, TN> },

static const KernelEntry kSigned[] = { ABQ_TILED_VARIANTS(ABQ_ENTRY_T) };
static const KernelEntry kUnsigned[] = { ABQ_TILED_VARIANTS(ABQ_ENTRY_F) };

#define ABQ_CAT_(a, b, c, d) a##b##c##d
#define ABQ_CAT(a, b, c, d) ABQ_CAT_(a, b, c, d)

void ABQ_CAT(abq_tiled_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSigned, (int)(sizeof(kSigned) / sizeof(kSigned[0])) };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsigned, (int)(sizeof(kUnsigned) / sizeof(kUnsigned[0])) };
}

} // namespace abq
