// GEMM core, VALU strategy: AND + popcount on the packed planes as they are (the reference's wire format,
// nothing prepared, nothing expanded), K along the lanes, wavefront reduction.  Meant for decode-sized M.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for one (x_bits, w_bits) pair per
// translation unit: compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>.
//
// Work split.  LPR = 2^lpr_log2 lanes share one weight row, so a wave covers 64 / LPR rows and a
// workgroup of eight waves 8 * 64 / LPR rows; lane c of a row handles the 16-byte units c, c + LPR, ...
// of that row (a unit is four plane words = 128 K elements of one plane).  The activation planes of the
// workgroup's MT rows go from global memory straight into LDS once (global_load_lds_dwordx4: no registers,
// no wait before the weight loads are issued) and are read from there with ds_read_b128, whichever
// weight row a lane works on.  Every weight word is read exactly once, with 16-byte loads issued from
// inline assembly right behind the activation loads (plain loads would be sunk below the barrier by the
// compiler): D passes of P planes per lane are in flight before the first wait, one counted wait and
// one barrier later the popcounts start.  Per unit, plane pair and activation row a lane does
// 4 v_and + 4 v_bcnt (chained through the accumulate operand of v_bcnt); the plane-pair counts are
// combined with their weights +/-2^(i+j) once at the end when there are few of them (registers), else
// with a multiply-add per unit.  The LPR partial sums meet through DPP row operations (and one or two
// cross-row shuffles): no LDS traffic for the reduction.
#include "abq_kernels.h"

#ifndef ABQ_Q
#error "compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>"
#endif

namespace abq {

typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr int kBcntWaves = 8;

__device__ __forceinline__ void bc_load_to_lds(const void *src, unsigned lds_addr)
{
    // lane l of the wave lands at lds_addr + 16 * l (M0 cannot be named as clobbered: the compiler reserves it)
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(src)
                 : "memory");
}

__device__ __forceinline__ v4u bc_load16(const char *base, uint32_t off)
{
    v4u v;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(v) : "v"(off), "s"(base) : "memory");
    return v;
}

__device__ __forceinline__ void bc_wait_loads_n(int n)
{
    switch (n) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    case 14: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
    case 16: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
    default:
        // a smaller count than needed only waits longer
        if (n > 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else if (n > 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        break;
    }
}
// ties a register filled by bc_load16 to the wait in front of it: every use comes after
__device__ __forceinline__ void bc_landed(v4u &v) { asm volatile("" : "+v"(v)); }

// popcount(x & w) over four words, added to acc (v_bcnt_u32_b32 adds its second operand)
__device__ __forceinline__ int popc4_acc(const v4u &x, const v4u &w, int acc)
{
    acc += __builtin_popcount(x[0] & w[0]);
    acc += __builtin_popcount(x[1] & w[1]);
    acc += __builtin_popcount(x[2] & w[2]);
    acc += __builtin_popcount(x[3] & w[3]);
    return acc;
}

template <int CTRL> __device__ __forceinline__ int bc_dpp_add(int v)
{
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}

// D: passes of a lane whose loads are in flight together (a pass = one unit of each of the P planes)
template <int Q, int P, bool SIGNED, int MT, int D>
__global__ __launch_bounds__(64 * kBcntWaves) void gemm_bcnt(const GemmArgs a)
{
    constexpr int NT = 64 * kBcntWaves;
    constexpr bool PAIRS = Q * P * MT <= 64; // one counter per plane pair and row, weighted at the end
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lpr_log2 = a.lpr_log2;
    const int LPR = 1 << lpr_log2;
    const int M = a.M, N = a.N, KW = a.KW;
    const int units = KW >> 2;
    const int m0 = blockIdx.y * MT;
    const int Mb = min(MT, M - m0);
    const int lir = lane & (LPR - 1);
    const int row = (blockIdx.x * kBcntWaves + wid) * (64 >> lpr_log2) + (lane >> lpr_log2);
    const unsigned xs_addr = (unsigned)(size_t)smem;
    const char *Xg = reinterpret_cast<const char *>(a.X);
    const char *Wg = reinterpret_cast<const char *>(a.W);

    // ---- activation planes of rows m0 .. m0 + Mb - 1 -> LDS [Q][Mb][KW] ---------------------------------
    const int per_plane = Mb * units;      // 16-byte chunks per plane
    const int xchunks = Q * per_plane;
    if (Mb == M) { // all planes are one contiguous block
        for (int pb = wid * 64; pb < xchunks; pb += NT) {
            const int p = min(pb + lane, xchunks - 1);
            bc_load_to_lds(Xg + (uint32_t)p * 16u, xs_addr + (unsigned)pb * 16u);
        }
    } else {
        for (int pb = wid * 64; pb < xchunks; pb += NT) {
            const int p = min(pb + lane, xchunks - 1);
            const int i = p / per_plane, c = p - i * per_plane;
            bc_load_to_lds(Xg + ((size_t)(i * M + m0) * KW) * 4 + (size_t)c * 16, xs_addr + (unsigned)pb * 16u);
        }
    }

    // ---- weights: plane j of (row, unit u) at j * plane_bytes + row_off + 16 u -----------------------------
    const uint32_t row_off = (uint32_t)min(row, N - 1) * (uint32_t)KW * 4u;
    const size_t plane_bytes = (size_t)N * KW * 4;

    int cnt[PAIRS ? MT * Q * P : 1];
    int acc[MT];
#pragma unroll
    for (int i = 0; i < (PAIRS ? MT * Q * P : 1); ++i)
        cnt[i] = 0;
#pragma unroll
    for (int t = 0; t < MT; ++t)
        acc[t] = 0;

    int round = 0;
    do {
        v4u wv[D][P];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int u = min(lir + (round * D + d) * LPR, units - 1); // units past the end repeat the last one (not used)
#pragma unroll
            for (int j = 0; j < P; ++j)
                wv[d][j] = bc_load16(Wg + j * plane_bytes, row_off + (uint32_t)u * 16u);
        }
        if (round == 0) {
            bc_wait_loads_n(D * P); // the activation loads are older than these
            __syncthreads();
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int u = lir + (round * D + d) * LPR;
            // waited for and marked as landed on every path: a register with a load in flight must not look free
            bc_wait_loads_n((D - 1 - d) * P);
#pragma unroll
            for (int j = 0; j < P; ++j)
                bc_landed(wv[d][j]);
            if (u < units) {
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    if (t < Mb) { // uniform
#pragma unroll
                        for (int i = 0; i < Q; ++i) {
                            const v4u x = *reinterpret_cast<const v4u *>(smem + ((size_t)(i * Mb + t) * KW) * 4 + (size_t)u * 16);
#pragma unroll
                            for (int j = 0; j < P; ++j) {
                                if (PAIRS)
                                    cnt[(t * Q + i) * P + j] = popc4_acc(x, wv[d][j], cnt[(t * Q + i) * P + j]);
                                else
                                    acc[t] += popc4_acc(x, wv[d][j], 0) * plane_pair_weight(i, j, Q, P, SIGNED);
                            }
                        }
                    }
                }
            }
        }
        ++round;
    } while ((round * D) * LPR < units);

    if (PAIRS) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < Q; ++i)
#pragma unroll
                for (int j = 0; j < P; ++j)
                    acc[t] += cnt[(t * Q + i) * P + j] * plane_pair_weight(i, j, Q, P, SIGNED);
    }

    // ---- the LPR partial sums of a row meet: butterflies inside a row of sixteen lanes with DPP, across rows with shuffles
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        int v = acc[t];
        v = bc_dpp_add<0xB1>(v);  // quad_perm [1,0,3,2]
        v = bc_dpp_add<0x4E>(v);  // quad_perm [2,3,0,1]
        v = bc_dpp_add<0x141>(v); // row_half_mirror: the other quad of the half row
        v = bc_dpp_add<0x140>(v); // row_mirror: the other half row
        if (LPR > 16)
            v += __shfl_xor(v, 16, 64);
        if (LPR > 32)
            v += __shfl_xor(v, 32, 64);
        acc[t] = v;
    }
    if (lir == 0 && row < N) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
            if (t < Mb)
                store_result(a, m0 + t, row, acc[t]);
    }
}

template <int Q, int P, bool SIGNED, int MT, int D>
static hipError_t launch_bcnt(const GemmArgs &a, hipStream_t stream)
{
    const int rpw = 64 >> a.lpr_log2;
    const int rows_per_wg = kBcntWaves * rpw;
    const int mb = a.M < MT ? a.M : MT;
    const size_t lds = (size_t)Q * mb * a.KW * 4 + 1024; // whole wave loads: up to 63 chunks of slack
    if (lds > 160 * 1024 || (size_t)a.N * a.KW * 4 >= (1ull << 32))
        return hipErrorInvalidValue;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_bcnt<Q, P, SIGNED, MT, D>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    const dim3 grid((a.N + rows_per_wg - 1) / rows_per_wg, (a.M + MT - 1) / MT);
    hipLaunchKernelGGL((gemm_bcnt<Q, P, SIGNED, MT, D>), grid, dim3(64 * kBcntWaves), lds, stream, a);
    return hipGetLastError();
}

// Native tile space of this strategy: activation rows per workgroup x passes in flight (the tuple's NSTAGE).
#define ABQ_BCNT_VARIANTS(V) V(1, 1) V(2, 1) V(4, 1) V(1, 3) V(2, 3) V(4, 3)

#define ABQ_ENTRY_T(MT, D) { 1, MT, 1, 1, kBcntWaves, 1, D, &launch_bcnt<ABQ_Q, ABQ_P, true, MT, D> },
#define ABQ_ENTRY_F(MT, D) { 1, MT, 1, 1, kBcntWaves, 1, D, &launch_bcnt<ABQ_Q, ABQ_P, false, MT, D> },

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
