// GEMM core for prefill-sized M on the FP6 matrix cores: a third route beside the popcount and
// int8 MFMA strategies, for operands that fit a 6-bit float exactly.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for every bit pair whose operands are
// unsigned of at most 4 bits or signed of at most 5 bits (w2a2 ... w5a5 signed, w2a2 ... w4a4
// unsigned, w2a4).
//
// Why it is exact.  CDNA4's v_mfma_f32_32x32x64_f8f6f4 multiplies FP6 (E2M3: sign, 2 exponent
// bits, 3 mantissa bits) operands at twice the int8 rate and accumulates in fp32.  Read with
// 1/8 as the unit, the E2M3 codes 0..15 of the subnormal range and the first binade are the
// integers 0..15 in plain binary, and 16 is 0b010000: a sign-magnitude integer of magnitude
// <= 16 IS its FP6 encoding.  Every product is a multiple of 1/64 and every partial sum is
// below 2^24 units as long as max|x| * max|w| * K < 2^24 (checked by the host), so the fp32
// accumulation never rounds and acc * 64 is the integer result, bit for bit.
//
// Operand format (library-private, written by relayout_planes_fp6_kernel): a row's K tile of 128
// elements is one record of 96 bytes = four 192-bit strings of 32 six-bit codes; strings 0 and 1
// feed lanes 0-31 of the two MFMA K steps of the tile, strings 2 and 3 lanes 32-63, so a lane
// fetches both steps with three aligned ds_read_b128.  Records are stored tiled[kt][row][96 B].
//
// Nothing is unpacked in this kernel, and the tiles never pass through registers on their way
// in: the load unit writes them from global memory straight into LDS (global_load_lds_dwordx4),
// S stages deep; the waves read their MFMA fragments out of LDS one tile ahead of the MFMAs that
// use them.  One barrier per K tile; workgroup -> tile mapping keeps a band of N per XCD as in
// the int8 tiled kernel.  What bounds it on LLaMA-sized problems is the rate at which L2 delivers
// the tiles (about 22 TB/s over the chip), not the matrix cores.
#include "abq_kernels.h"

namespace abq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4))); // a 16-byte piece (a native vector: copies stay in registers)

constexpr int kFp6Units = 6;      // 16-byte units per record
constexpr int kFp6LdsRow = 96;    // bytes per row in LDS: the records as they are, no padding

// LDS placement of 16-byte unit `pos` of an operand block (pos = row * 6 + unit): the records as
// they are, with units swapped in pairs inside every second 256-byte line.  The fragment reads
// (sixteen lanes = sixteen consecutive rows, same unit: positions 6 apart, which alone would meet
// in pairs eight rows = three lines apart) then hit sixteen different bank groups, and a run of 64
// consecutive units still fills 64 consecutive places.  The function is its own inverse.
__device__ __forceinline__ int fp6_lds_offset(int pos) { return (pos ^ ((pos >> 4) & 1)) * 16; }

// global_load_lds_dwordx4 writes a wave's 64 x 16 bytes straight into LDS (at M0 + 16 * lane): no
// register staging, no ds_write instructions (LDS stores run at a third of the LDS read rate on
// this chip), and the data never crosses the vector register file.  Tile t + S - 1 is requested
// during tile t into the stage tile t - 1 occupied.  The compiler would drain every outstanding
// load of this kind before each ds_read, so they are issued from inline assembly and waited for
// by hand: every wave issues the same number of loads per tile, which makes "all but the newest
// n tiles have landed" one s_waitcnt vmcnt(n * loads per tile).  No other vector-memory
// instruction may be in flight while that count is relied on: the kernel has none inside its K
// loop and drains the counter before its epilogue.
template <int N> __device__ __forceinline__ void fp6_wait_loads()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void fp6_load_to_lds(const v4u *src, unsigned lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "memory");
}

template <int TM, int TN, int WM, int WN, int S>
__global__ __launch_bounds__(64 * WM * WN, (WM * WN > 4 || TM * TN > 4) ? 1 : 2)
void gemm_mfma_fp6(const GemmArgs a, const v4u *xt, const v4u *wt, int m_blocks, int n_blocks_per_xcd)
{
    constexpr int NW = WM * WN;
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr int BUF_BYTES = (BM + BN) * kFp6LdsRow;
    constexpr int NIA = BM * kFp6Units / 64;             // wave loads of 1 KiB per tile: activations
    constexpr int NI = (BM + BN) * kFp6Units / 64;       // ... and in all
    constexpr int NPW = (NI + NW - 1) / NW;              // per wave
    static_assert(S >= 3 && S <= 4, "three or four LDS stages");
    static_assert(NPW * (S - 1) < 64, "the load counter has six bits");

    extern __shared__ __align__(16) unsigned char smem[]; // [S][BM + BN][96]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wid / WN, wn = wid % WN;
    const int r = lane & 31, g = lane >> 5;
    const int M = __builtin_amdgcn_readfirstlane(a.M), N = __builtin_amdgcn_readfirstlane(a.N);
    const int ktiles = __builtin_amdgcn_readfirstlane(a.K) / 128;

    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int nb = xcd * n_blocks_per_xcd + slot / m_blocks;
    const int mb = slot % m_blocks;
    const int m0 = mb * BM, n0 = nb * BN;
    if (n0 >= N)
        return; // uniform over the workgroup, before any barrier

    // Wave load q of a tile fills LDS units [64 q, 64 q + 64) of the stage; the unit at LDS position P
    // is unit P ^ ((P >> 4) & 1) of the tile (fp6_lds_offset is its own inverse), activations first.
    // Loads past the last one repeat an earlier load of the wave (same data, same place), so that
    // every wave issues NPW loads per tile.
    uint32_t goff[NPW];     // 16-byte units from the start of the operand's records of one K tile
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
        int q = wid + NW * i;
        if (q >= NI)
            q -= NW;
        const int P = 64 * q + lane;
        const int u = P ^ ((P >> 4) & 1);
        const bool is_a = q < NIA; // wave-uniform
        const int v = is_a ? u : u - BM * kFp6Units;
        const int row = v / kFp6Units, col = v % kFp6Units;
        goff[i] = (uint32_t)(is_a ? min(m0 + row, M - 1) : min(n0 + row, N - 1)) * kFp6Units + col;
    }
    const size_t stride_a = (size_t)M * kFp6Units, stride_b = (size_t)N * kFp6Units;
    const unsigned lds0 = (unsigned)(size_t)smem; // LDS byte address of the first stage

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[i][j][e] = 0.f;

    unsigned char *lds_a = smem;
    unsigned char *lds_b = smem + BM * kFp6LdsRow;
    int a_off[3], b_off[3];
#pragma unroll
    for (int q = 0; q < 3; ++q) {
        a_off[q] = fp6_lds_offset((wm * 32 * TM + r) * kFp6Units + 3 * g + q);
        b_off[q] = fp6_lds_offset((wn * 32 * TN + r) * kFp6Units + 3 * g + q);
    }
    static_assert(BUF_BYTES % 512 == 0, "stages keep the line parity");
    // Fragment sets as the raw 16-byte reads: piece 3 f + c is read c of fragment f (activation
    // fragments first), and the MFMA operands are cut out of them when they are used.
    constexpr int NF = TM + TN, NR = 3 * NF, NM = 2 * TM * TN;
    v4i q0[NR], q1[NR];
    auto read_piece = [&](v4i(&q)[NR], int stage, int p) {
        const int f = p / 3, c = p % 3;
        q[p] = f < TM ? *reinterpret_cast<const v4i *>(lds_a + stage + f * 32 * kFp6LdsRow + a_off[c])
                      : *reinterpret_cast<const v4i *>(lds_b + stage + (f - TM) * 32 * kFp6LdsRow + b_off[c]);
    };
    auto operand = [&](const v4i(&q)[NR], int f, int ks) -> v8i {
        // dwords 0-5 of the 12 a lane holds are the first K step's operand, 6-11 the second's
        return ks == 0 ? __builtin_shufflevector(q[3 * f], q[3 * f + 1], 0, 1, 2, 3, 4, 5, -1, -1)
                       : __builtin_shufflevector(q[3 * f + 1], q[3 * f + 2], 2, 3, 4, 5, 6, 7, -1, -1);
    };
    auto request = [&](int kt_req, int stage, int i) {
        const int kn = min(kt_req, ktiles - 1);
        int q = wid + NW * i;
        if (q >= NI)
            q -= NW;
        fp6_load_to_lds((q < NIA ? xt + kn * stride_a : wt + kn * stride_b) + goff[i], lds0 + stage + q * 1024);
    };

    // prologue: tiles 0 .. S-2 requested; tile 0 read into the first fragment set; tile 1 landed
#pragma unroll
    for (int s = 0; s < S - 1; ++s)
#pragma unroll
        for (int i = 0; i < NPW; ++i)
            request(s, s * BUF_BYTES, i);
    fp6_wait_loads<NPW * (S - 2)>();
    __syncthreads();
#pragma unroll
    for (int p = 0; p < NR; ++p)
        read_piece(q0, 0, p);
    fp6_wait_loads<NPW * (S - 3)>();
    __syncthreads();

    int st_req = (S - 1) * BUF_BYTES; // stage the next request goes to: the one tile t - 1 occupied
    int st_rd = BUF_BYTES;            // stage of tile t + 1
    // One K tile.  On entry every wave's share of tile KT + 1 has landed (wait + barrier at the end of
    // the previous tile), and the fragment set QC holds tile KT.  The wave's load requests and LDS reads
    // are dealt out between its MFMAs: a wave issues in order, and a burst of requests at the top of
    // the tile would hold its MFMAs back until the load unit and the LDS have taken the whole burst.
#define ABQ_FP6_K_TILE(KT, QC, QN)                                                                              \
    {                                                                                                           \
        _Pragma("unroll") for (int k = 0; k < NM; ++k)                                                          \
        {                                                                                                       \
            const int ks = k / (TM * TN), i = (k / TN) % TM, j = k % TN;                                        \
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(operand(QC, i, ks), operand(QC, TM + j, ks), \
                                                                       acc[i][j], 2, 2, 0, 0, 0, 0);            \
            _Pragma("unroll") for (int d = k * NPW / NM; d < (k + 1) * NPW / NM; ++d)                           \
                request((KT) + S - 1, st_req, d);                                                               \
            _Pragma("unroll") for (int p = k * NR / NM; p < (k + 1) * NR / NM; ++p)                             \
                read_piece(QN, st_rd, p);                                                                       \
            __builtin_amdgcn_sched_barrier(0);                                                                  \
        }                                                                                                       \
        st_req = st_req + BUF_BYTES == S * BUF_BYTES ? 0 : st_req + BUF_BYTES;                                  \
        st_rd = st_rd + BUF_BYTES == S * BUF_BYTES ? 0 : st_rd + BUF_BYTES;                                     \
        fp6_wait_loads<NPW * (S - 3)>(); /* tile KT + 2 has landed; KT + 3 (four stages) may still fly */       \
        __syncthreads();                                                                                        \
    }

    int kt = 0;
    for (; kt + 2 <= ktiles; kt += 2) {
        ABQ_FP6_K_TILE(kt, q0, q1)
        ABQ_FP6_K_TILE(kt + 1, q1, q0)
    }
    if (kt < ktiles)
        ABQ_FP6_K_TILE(kt, q0, q1)
#undef ABQ_FP6_K_TILE
    fp6_wait_loads<0>(); // the clamped requests past the last tile: nothing of ours may be in flight below

    const StoreOperands so = store_operands(a);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * 32 * TN + j * 32 + r;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4);
                const int v = (int)(acc[i][j][e] * 64.0f);
                if (m < M && n < N)
                    store_result_compact(so, m, n, v);
            }
        }
    }
}

template <int TM, int TN, int WM, int WN> static hipError_t launch_mfma_fp6(const GemmArgs &a, hipStream_t stream)
{
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    const int m_blocks = (a.M + BM - 1) / BM, n_blocks = (a.N + BN - 1) / BN;
    const int npx = (n_blocks + 7) / 8;
    const dim3 grid(8 * npx * m_blocks);
    // four LDS stages (three tiles of loads in flight), except for the 128 x 128 tile, which keeps two
    // workgroups on a compute unit with three
    constexpr int S = (TM == 2 && TN == 2 && WM == 2 && WN == 2) ? 3 : 4;
    const size_t lds = S * (size_t)(BM + BN) * kFp6LdsRow;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_fp6<TM, TN, WM, WN, S>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    hipLaunchKernelGGL((gemm_mfma_fp6<TM, TN, WM, WN, S>), grid, dim3(64 * WM * WN), lds, stream, a,
                       reinterpret_cast<const v4u *>(a.X), reinterpret_cast<const v4u *>(a.W), m_blocks, npx);
    return hipGetLastError();
}

// Tile space: MFMA tiles per wave (TM, TN) and waves along M, N; nstage 5 marks the FP6 records.
#define ABQ_FP6_VARIANTS(V) V(2, 2, 4, 2) V(4, 2, 2, 2) V(2, 2, 2, 2) V(2, 1, 2, 2) V(1, 1, 2, 2)
#define ABQ_FP6_ENTRY(TM, TN, WM, WN) { 32, TM, TN, WM, WN, 1, 5, &launch_mfma_fp6<TM, TN, WM, WN>, 128 },
static const KernelEntry kFp6Entries[] = { ABQ_FP6_VARIANTS(ABQ_FP6_ENTRY) };

const KernelEntry *fp6_entries(int *count)
{
    *count = (int)(sizeof(kFp6Entries) / sizeof(kFp6Entries[0]));
    return kFp6Entries;
}

} // namespace abq
