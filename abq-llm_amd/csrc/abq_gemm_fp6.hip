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
// Nothing is unpacked in this kernel: global -> registers -> LDS (the records as they are, 16-byte
// units swapped in pairs in every second 256-byte line: conflict free for b128 writes and reads) -> MFMA.  LDS is double buffered, one barrier per K tile; workgroup -> tile
// mapping keeps a band of N per XCD as in the int8 tiled kernel.
#include "abq_kernels.h"

namespace abq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4))); // a 16-byte piece (a native vector: copies stay in registers)

constexpr int kFp6Units = 6;      // 16-byte units per record
constexpr int kFp6LdsRow = 96;    // bytes per row in LDS: the records as they are, no padding

// LDS placement of 16-byte unit `pos` of an operand block (pos = row * 6 + unit): units are swapped
// in pairs inside every second 256-byte line.  A wave's global load of 64 consecutive units then
// lands as four conflict-free ds_write_b128 (each group of sixteen lanes fills one line), and the
// fragment reads (sixteen lanes = sixteen consecutive rows, same unit: positions 6 apart, which
// alone would meet in pairs eight rows = three lines apart) hit sixteen different bank groups.
__device__ __forceinline__ int fp6_lds_offset(int pos) { return (pos ^ ((pos >> 4) & 1)) * 16; }

// One lane's share of a 32-row fragment for both K steps of a tile: 48 bytes, three ds_read_b128.
__device__ __forceinline__ void load_fragment(v8i (&f)[2], const unsigned char *base, const int (&off)[3])
{
    const v4i q0 = *reinterpret_cast<const v4i *>(base + off[0]);
    const v4i q1 = *reinterpret_cast<const v4i *>(base + off[1]);
    const v4i q2 = *reinterpret_cast<const v4i *>(base + off[2]);
    const v8i lo = __builtin_shufflevector(q0, q1, 0, 1, 2, 3, 4, 5, 6, 7);
    const v8i hi = __builtin_shufflevector(q1, q2, 2, 3, 4, 5, 6, 7, -1, -1);
    f[0] = __builtin_shufflevector(lo, lo, 0, 1, 2, 3, 4, 5, -1, -1);
    f[1] = hi;
}

// This thread's share of one operand's tile: pieces of 16 bytes, piece p = tid + NT * i
// (ROWS is a multiple of 32).
template <int ROWS, int NT> struct Fp6Stage {
    static constexpr int kPieces = ROWS * kFp6Units;
    static constexpr int NP = (kPieces + NT - 1) / NT;
    static constexpr bool kRagged = kPieces % NT != 0;

    // offsets of the pieces: `g` in 16-byte units from the start of a K tile's records, `l` in bytes
    // from the start of the operand's block in LDS (negative: the thread has no such piece)
    static __device__ __forceinline__ void offsets(int tid, int row0, int rows, uint32_t (&g)[NP], int (&l)[NP])
    {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int p = tid + NT * i; // consecutive lanes, consecutive units: a wave loads 1 KiB in one piece
            const int rr = p / kFp6Units, u = p % kFp6Units;
            const bool have = !kRagged || i + 1 < NP || p < kPieces;
            g[i] = (uint32_t)min(row0 + (have ? rr : 0), rows - 1) * kFp6Units + u;
            l[i] = have ? fp6_lds_offset(p) : -1;
        }
    }
    static __device__ __forceinline__ void load(v4u (&r)[NP], const v4u *tile, const uint32_t (&g)[NP])
    {
#pragma unroll
        for (int i = 0; i < NP; ++i)
            r[i] = tile[g[i]];
    }
    static __device__ __forceinline__ void store(const v4u (&r)[NP], unsigned char *lds, const int (&l)[NP])
    {
#pragma unroll
        for (int i = 0; i < NP; ++i)
            if (!kRagged || i + 1 < NP || l[i] >= 0)
                *reinterpret_cast<v4u *>(lds + l[i]) = r[i];
    }
};

template <int TM, int TN, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN, (WM * WN > 4 || TM * TN > 4) ? 1 : 2)
void gemm_mfma_fp6(const GemmArgs a, const v4u *xt, const v4u *wt, int m_blocks, int n_blocks_per_xcd)
{
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr int BUF_BYTES = (BM + BN) * kFp6LdsRow;
    using StageA = Fp6Stage<BM, NT>;
    using StageB = Fp6Stage<BN, NT>;

    extern __shared__ __align__(16) unsigned char smem[]; // [2][BM + BN][96]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = tid >> 6;
    const int wm = wid / WN, wn = wid % WN;
    const int r = lane & 31, g = lane >> 5;
    const int M = __builtin_amdgcn_readfirstlane(a.M), N = __builtin_amdgcn_readfirstlane(a.N);
    const int ktiles = __builtin_amdgcn_readfirstlane(a.K) / 128;

    // workgroup -> tile: XCD x = id % 8 owns n blocks [x * npx, (x+1) * npx), M fastest
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int nb = xcd * n_blocks_per_xcd + slot / m_blocks;
    const int mb = slot % m_blocks;
    const int m0 = mb * BM, n0 = nb * BN;
    if (n0 >= N)
        return; // uniform over the workgroup, before any barrier

    uint32_t ga[StageA::NP], gb[StageB::NP];
    int la[StageA::NP], lb[StageB::NP];
    StageA::offsets(tid, m0, M, ga, la);
    StageB::offsets(tid, n0, N, gb, lb);
    const size_t stride_a = (size_t)M * kFp6Units, stride_b = (size_t)N * kFp6Units; // 16-byte units per K tile

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
    // Software pipeline.  While the MFMAs of tile t run out of one set of fragment registers, the
    // ds_reads of tile t + 1 fill the other set, tiles t + 2 .. t + D wait in register slots (tile
    // t + 2 is written to LDS at the end of tile t, into the buffer tile t occupied) and the global
    // loads of tile t + 1 + D are issued into the slot tile t + 1 left: D - 1 whole K tiles of MFMAs
    // hide a load.  Everything is unrolled (by six for three slots) with named arrays, so every
    // register index is a constant.  Tiles past the end
    // are clamped to the last one: their copies land in buffers and registers nobody uses again.
    v4u ra0[StageA::NP], rb0[StageB::NP], ra1[StageA::NP], rb1[StageB::NP], ra2[StageA::NP], rb2[StageB::NP];
    v8i fa0[TM][2], fb0[TN][2], fa1[TM][2], fb1[TN][2];
    // this lane's three units of a fragment row; 32 rows further on (192 units = 12 lines) and in the other
    // buffer (a multiple of two lines) the placement repeats, so those offsets are plain constants
    int a_off[3], b_off[3];
#pragma unroll
    for (int q = 0; q < 3; ++q) {
        a_off[q] = fp6_lds_offset((wm * 32 * TM + r) * kFp6Units + 3 * g + q);
        b_off[q] = fp6_lds_offset((wn * 32 * TN + r) * kFp6Units + 3 * g + q);
    }
    static_assert((32 * kFp6LdsRow) % 512 == 0, "fragment rows and buffers keep the line parity");
#define ABQ_FP6_LOAD(KT, RA, RB)                               \
    {                                                          \
        const int kn_ = min((KT), ktiles - 1);                 \
        StageA::load(RA, xt + kn_ * stride_a, ga);             \
        StageB::load(RB, wt + kn_ * stride_b, gb);             \
    }
    // a lane's 48 bytes land in twelve consecutive registers: dwords 0-5 are the operand of the first
    // K step, 6-11 of the second (the two upper dwords of the 8-dword operand are not read)
#define ABQ_FP6_READ(FA, FB, BUF)                                                   \
    {                                                                               \
        _Pragma("unroll") for (int i = 0; i < TM; ++i)                              \
            load_fragment(FA[i], lds_a + (BUF) + i * 32 * kFp6LdsRow, a_off);       \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                              \
            load_fragment(FB[j], lds_b + (BUF) + j * 32 * kFp6LdsRow, b_off);       \
    }
    // D register slots: three where the registers allow it (eight waves share the tile: 20 registers a
    // slot), two otherwise
    constexpr int D = WM * WN > 4 ? 3 : 2;
    ABQ_FP6_LOAD(0, ra0, rb0)
    ABQ_FP6_LOAD(1, ra1, rb1)
    if (D == 3)
        ABQ_FP6_LOAD(2, ra2, rb2)
    StageA::store(ra0, lds_a, la);
    StageB::store(rb0, lds_b, lb);
    ABQ_FP6_LOAD(D, ra0, rb0) // tile D into slot D % D = 0
    StageA::store(ra1, lds_a + BUF_BYTES, la);
    StageB::store(rb1, lds_b + BUF_BYTES, lb);
    __syncthreads();
    ABQ_FP6_READ(fa0, fb0, 0)
    __syncthreads(); // every wave holds its fragments of tile 0 before buffer 0 is written again

    // One K tile.  On entry buffer (KT + 1) % 2 holds tile KT + 1 and the fragments FCA / FCB hold tile KT.
#define ABQ_FP6_K_TILE(KT, FCA, FCB, FNA, FNB, RAL, RBL, RAS, RBS)                                              \
    {                                                                                                           \
        const int buf = ((KT) & 1) * BUF_BYTES;                                                                 \
        ABQ_FP6_LOAD((KT) + 1 + D, RAL, RBL)                                                                    \
        __builtin_amdgcn_sched_barrier(0); /* the loads leave first: a whole tile of MFMAs hides them */        \
        ABQ_FP6_READ(FNA, FNB, BUF_BYTES - buf)                                                                 \
        _Pragma("unroll") for (int ks = 0; ks < 2; ++ks)                                                        \
            _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                      \
                _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                  \
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(FCA[i][ks], FCB[j][ks], acc[i][j], \
                                                                               2, 2, 0, 0, 0, 0);               \
        StageA::store(RAS, lds_a + buf, la);                                                                    \
        StageB::store(RBS, lds_b + buf, lb);                                                                    \
        __syncthreads(); /* waits for this wave's ds_reads and ds_writes, then for the other waves */           \
    }

    // fragment sets alternate (period 2), register slots rotate (period 3): six tiles per round
#define ABQ_FP6_T0(KT) ABQ_FP6_K_TILE(KT, fa0, fb0, fa1, fb1, ra1, rb1, ra2, rb2)
#define ABQ_FP6_T1(KT) ABQ_FP6_K_TILE(KT, fa1, fb1, fa0, fb0, ra2, rb2, ra0, rb0)
#define ABQ_FP6_T2(KT) ABQ_FP6_K_TILE(KT, fa0, fb0, fa1, fb1, ra0, rb0, ra1, rb1)
#define ABQ_FP6_T3(KT) ABQ_FP6_K_TILE(KT, fa1, fb1, fa0, fb0, ra1, rb1, ra2, rb2)
#define ABQ_FP6_T4(KT) ABQ_FP6_K_TILE(KT, fa0, fb0, fa1, fb1, ra2, rb2, ra0, rb0)
#define ABQ_FP6_T5(KT) ABQ_FP6_K_TILE(KT, fa1, fb1, fa0, fb0, ra0, rb0, ra1, rb1)
    int kt = 0;
    if (D == 3) {
        for (; kt + 6 <= ktiles; kt += 6) {
            ABQ_FP6_T0(kt)
            ABQ_FP6_T1(kt + 1)
            ABQ_FP6_T2(kt + 2)
            ABQ_FP6_T3(kt + 3)
            ABQ_FP6_T4(kt + 4)
            ABQ_FP6_T5(kt + 5)
        }
        if (kt < ktiles) { // up to five tiles are left
            ABQ_FP6_T0(kt)
            if (kt + 1 < ktiles) {
                ABQ_FP6_T1(kt + 1)
                if (kt + 2 < ktiles) {
                    ABQ_FP6_T2(kt + 2)
                    if (kt + 3 < ktiles) {
                        ABQ_FP6_T3(kt + 3)
                        if (kt + 4 < ktiles)
                            ABQ_FP6_T4(kt + 4)
                    }
                }
            }
        }
    } else {
        // two slots: tile t + 2 is written from slot t % 2 while tile t + 3 loads into slot (t + 1) % 2
        for (; kt + 2 <= ktiles; kt += 2) {
            ABQ_FP6_K_TILE(kt, fa0, fb0, fa1, fb1, ra1, rb1, ra0, rb0)
            ABQ_FP6_K_TILE(kt + 1, fa1, fb1, fa0, fb0, ra0, rb0, ra1, rb1)
        }
        if (kt < ktiles)
            ABQ_FP6_K_TILE(kt, fa0, fb0, fa1, fb1, ra1, rb1, ra0, rb0)
    }
#undef ABQ_FP6_T0
#undef ABQ_FP6_T1
#undef ABQ_FP6_T2
#undef ABQ_FP6_T3
#undef ABQ_FP6_T4
#undef ABQ_FP6_T5
#undef ABQ_FP6_K_TILE
#undef ABQ_FP6_READ
#undef ABQ_FP6_LOAD

    const StoreOperands so = store_operands(a);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * 32 * TN + j * 32 + r;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4);
                // both operands carry 1/8 as their unit: the sum is the integer result / 64, exactly
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
    const size_t lds = 2 * (size_t)(BM + BN) * kFp6LdsRow;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_fp6<TM, TN, WM, WN>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    const dim3 grid(8 * npx * m_blocks);
    hipLaunchKernelGGL((gemm_mfma_fp6<TM, TN, WM, WN>), grid, dim3(64 * WM * WN), lds, stream, a,
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
