// GEMM core for prefill-sized M: matrix-core strategy, LDS-staged, operands in the K-tiled
// plane layout.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for one (x_bits, w_bits) pair per
// translation unit: compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>.
//
// Why a second layout.  In the reference layout a K tile of 128 elements is 16 bytes per
// (row, plane) and rows are K/8 bytes apart, so a workgroup tile touches one 128-byte cache line
// per 16 useful bytes; and turning plane words into int8 costs a bit-matrix transpose per 32
// elements, paid again by every workgroup that uses the row: the vector ALUs, not the matrix
// cores, then bound the kernel.  The K-tiled layout keeps the same number of bits as records
//     tiled[kt][row][BITS * 4 words],  kt = K tile of 128 elements,
// so the rows of a tile are contiguous and every line is used in full, and inside a record the
// bits are grouped into 4-, 2- and 1-bit fields (abq_bits.h) that unpack to int8 with one or
// two instructions per four elements.  Weights are converted once (they are static),
// activations once per call; see relayout_planes_kernel.
//
// Work split.  256 threads = 2 x 2 waves; a wave owns TM x TN MFMA tiles of 32 x 32, the
// workgroup tile is (64*TM) x (64*TN), the K tile 128.  Per K tile each thread unpacks TM
// word-sets (32 K elements each) of one activation row and TN of one weight row to int8
// and writes them to LDS, so every row is expanded once per workgroup and all
// threads do the same amount of work without divergence; the waves read their MFMA
// operands with ds_read_b128 (row stride 144 bytes: conflict free).  LDS is double buffered
// and the plane words of the next two K tiles are in flight in registers, so the expansion
// of tile i+1 and the loads of tile i+2 overlap the MFMAs of tile i; one barrier per K tile.
// Workgroups are numbered so that the 8 XCDs (workgroup id modulo 8) each work on a
// contiguous band of N, in groups of four m blocks (tile_of_workgroup): the workgroups an XCD
// runs at a time share their activation and weight blocks in that XCD's L2.
#include "abq_kernels.h"
#include "abq_gemm_staged.h"

#ifndef ABQ_Q
#error "compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>"
#endif

namespace abq {


constexpr int kTileK = 128;        // K elements per tile
constexpr int kLdsRow = 144;       // bytes per expanded row in LDS (128 + 16 padding)

// Loads the fields of WPT consecutive word-sets of one row of one K tile (field-packed layout,
// abq_bits.h) into dst = [4-bit field: 4*WPT words][2-bit: 2*WPT][1-bit: WPT].
template <int N> __device__ __forceinline__ void load_words(uint32_t *dst, const uint32_t *src)
{
    if (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) {
            const uint4 v = reinterpret_cast<const uint4 *>(src)[i];
            dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
        }
    } else if (N == 2) {
        const uint2 v = *reinterpret_cast<const uint2 *>(src);
        dst[0] = v.x; dst[1] = v.y;
    } else {
        dst[0] = src[0];
    }
}

template <int BITS, int WPT>
__device__ __forceinline__ void load_tile_words(uint32_t (&dst)[BITS * WPT], const uint32_t *tiled, int rows, int row,
                                                int kt, int first_ws)
{
    const uint32_t *rec = tiled + ((size_t)kt * rows + row) * (BITS * 4);
    if constexpr (BITS == 8) {
        load_words<8 * WPT>(dst, rec + 8 * first_ws);
        return;
    }
    if constexpr ((BITS & 4) != 0)
        load_words<4 * WPT>(dst + field_list_index(BITS, 4) * WPT, rec + field_word_offset(BITS, 4) + 4 * first_ws);
    if constexpr ((BITS & 2) != 0)
        load_words<2 * WPT>(dst + field_list_index(BITS, 2) * WPT, rec + field_word_offset(BITS, 2) + 2 * first_ws);
    if constexpr ((BITS & 1) != 0)
        load_words<WPT>(dst + field_list_index(BITS, 1) * WPT, rec + field_word_offset(BITS, 1) + first_ws);
}

// Expands WPT word-sets (32 K elements each) of one row and writes the int8 values to LDS.
// SUM (unsigned operands only) also accumulates the sum of the values.
template <int BITS, int WPT, Int8Mode MODE, bool SUM>
__device__ __forceinline__ void expand_words_to_lds(const uint32_t (&raw)[BITS * WPT], unsigned char *lds, int &value_sum)
{
#pragma unroll
    for (int ws = 0; ws < WPT; ++ws) {
        uint32_t o[8];
        if (SUM) {
            expand_fields<BITS, WPT, kLow>(raw, ws, o);
            value_sum += expanded_byte_sum(o);
            if (MODE == kFlip) {
#pragma unroll
                for (int d = 0; d < 8; ++d)
                    o[d] ^= 0x80808080u;
            }
        } else {
            expand_fields<BITS, WPT, MODE>(raw, ws, o);
        }
        uint4 *dst = reinterpret_cast<uint4 *>(lds + ws * 32);
        dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
        dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
    }
}

// ---- a thread's share of one operand's K stage ------------------------------------------------
//
// Two mappings.  Row-wise (any bit width): thread t takes WPT consecutive word-sets of tile row
// t / TPR, loading each field's words for them.  Piece-wise (widths with a single field: 2, 4, 8
// bits, whole-record stages): the tile's records are one contiguous run of 16-byte pieces and
// thread t takes pieces t, t + NT, ...: every load instruction of a wave then covers 1 KiB of
// consecutive memory, which the L1 serves at about 1.4x the rate of the row-wise pattern (64
// bytes per lane, measured 24.6 against 17.4 TB/s over the chip).  A piece is a run of elements of
// one row (16 for 8 bits, 32 for 4, 64 for 2), unpacked by the same field routines.
template <int BITS, int ROWS, int NT, int KB, Int8Mode MODE, bool SUM> struct OperandStage {
    static constexpr int WSETS = KB / 32;
    static constexpr bool kPiece = KB == 128 && (BITS == 2 || BITS == 4 || BITS == 8) && (ROWS * BITS) % NT == 0;
    static constexpr int WPT = ROWS * WSETS / NT; // row-wise: word-sets per thread
    static constexpr int TPR = WSETS / (WPT ? WPT : 1);
    static constexpr int NP = kPiece ? ROWS * BITS / NT : 1; // piece-wise: pieces per thread
    static constexpr int kWords = kPiece ? 4 * NP : BITS * WPT;
    static constexpr int kSums = kPiece ? NP : 1;
    static_assert(kPiece || WPT == 1 || WPT == 2 || WPT == 4, "rows * KB / (32 * threads) in {1, 2, 4}");

    // tiled: the operand in the field-packed layout; rows: its row count; row0: first row of the tile
    static __device__ __forceinline__ void load(uint32_t (&dst)[kWords], const uint32_t *tiled, int rows, int row0,
                                                int tid, int stage)
    {
        if constexpr (kPiece) {
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int c = tid + NT * i;
                const int row = min(row0 + c / BITS, rows - 1);
                const uint4 v = *reinterpret_cast<const uint4 *>(tiled + (((size_t)stage * rows + row) * BITS + c % BITS) * 4);
                dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
            }
        } else {
            constexpr int SPR = kTileK / KB;
            const int row = min(row0 + tid / TPR, rows - 1);
            load_tile_words<BITS, WPT>(dst, tiled, rows, row, stage / SPR, (stage % SPR) * WSETS + (tid % TPR) * WPT);
        }
    }

    // lds: the operand's rows of the stage buffer ([ROWS][KB + 16] bytes); sums: value sums per row share
    static __device__ __forceinline__ void expand(const uint32_t (&raw)[kWords], unsigned char *lds, int tid,
                                                  int (&sums)[kSums], bool live)
    {
        constexpr int LDS_ROW = KB + 16;
        if constexpr (kPiece) {
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int c = tid + NT * i;
                unsigned char *dst = lds + (c / BITS) * LDS_ROW + (c % BITS) * (128 / BITS);
                const uint32_t piece[4] = { raw[4 * i], raw[4 * i + 1], raw[4 * i + 2], raw[4 * i + 3] };
                if constexpr (BITS == 8) { // 16 elements, the bytes themselves
                    uint32_t o[4];
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                        o[d] = piece[d] ^ (MODE == kFlip ? 0x80808080u : 0u);
                    if (SUM) {
                        uint32_t part = 0;
#pragma unroll
                        for (int d = 0; d < 4; ++d)
                            part = __builtin_amdgcn_sad_u8(piece[d], 0u, part); // sum of the four bytes
                        sums[i] += live ? (int)part : 0;
                    }
                    *reinterpret_cast<uint4 *>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
                } else { // one word-set of 4 bits (4 words) or two of 2 bits (2 words each)
                    constexpr int PW = 4 / BITS; // word-sets in the piece: 1 for 4 bits, 2 for 2 bits
                    int part = 0;
                    expand_words_to_lds<BITS, PW, MODE, SUM>(piece, dst, part);
                    if (SUM)
                        sums[i] += live ? part : 0;
                }
            }
        } else {
            int part = 0;
            expand_words_to_lds<BITS, WPT, MODE, SUM>(raw, lds + (tid / TPR) * LDS_ROW + (tid % TPR) * WPT * 32, part);
            if (SUM)
                sums[0] += live ? part : 0;
        }
    }

    // adds the thread's value sums to the per-row totals in LDS
    static __device__ __forceinline__ void flush_sums(int *rowsum, int tid, const int (&sums)[kSums])
    {
        if constexpr (kPiece) {
#pragma unroll
            for (int i = 0; i < NP; ++i)
                atomicAdd(&rowsum[(tid + NT * i) / BITS], sums[i]);
        } else {
            atomicAdd(&rowsum[tid / TPR], sums[0]);
        }
    }
};

// GROUPED: group-wise weight scales (group size 64 or 128 along K, w_scale[N][K/group]) and
// per-token activation scales, fp16 output.  The int32 accumulators then cover one scale group
// and are folded into fp32 accumulators with the group's scale at every group boundary
// (semantics: algorithm/quantize/quantizer.py:111-179 of the reference, scales per row of W
// after reshaping to [-1, group_size]).  Not available for 8-bit unsigned operands.
//
// KB: K elements per LDS stage, 128 (a whole record) or 64 (half a record: half the LDS per
// stage, so that the 128 x 256 tile still fits two workgroups per compute unit).
//
// WM x WN: waves per workgroup along M and N (2 x 2, or 4 x 2 / 4 x 4 for the large tiles that
// cut the L2 -> L1 traffic per MFMA).
template <int Q, int P, bool SIGNED, int TM, int TN, bool GROUPED, int KB, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN, (WM * WN > 4 ? 1 : (TM * TN <= 4 || KB == 64 ? 2 : 1)))
void gemm_mfma_tiled(const GemmArgs a, const uint32_t *xt, const uint32_t *wt, int m_blocks, int n_blocks_per_xcd)
{
    constexpr int NT = 64 * WM * WN; // threads
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr int WSETS = KB / 32;          // word-sets of a row per stage
    constexpr int SPR = kTileK / KB;        // stages per record
    constexpr int LDS_ROW = KB + 16;        // bytes per expanded row in LDS: ds_read_b128 conflict free
    static_assert(KB == 128 || KB == 64, "a stage is a record or half of one");
    static_assert(!GROUPED || KB == 128, "group scales are folded per 128-element stage");
    constexpr Int8Mode XMODE = Int8ModeOf<Q, SIGNED>::value;
    constexpr Int8Mode WMODE = Int8ModeOf<P, SIGNED>::value;
    constexpr bool NEED_SX = WMODE == kFlip; // see abq_gemm_mfma.hip
    constexpr bool NEED_SW = XMODE == kFlip;
    constexpr int BUF_BYTES = (BM + BN) * LDS_ROW;

    extern __shared__ __align__(16) unsigned char smem[];
    // [2][BM + BN][144] expanded rows, then row sums [BM + BN]
    int *rowsum = reinterpret_cast<int *>(smem + 2 * BUF_BYTES);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = tid >> 6;
    const int wm = wid / WN, wn = wid % WN;
    const int r = lane & 31, g = lane >> 5;
    // scalar copies of the shape: every branch on them below is a scalar branch
    const int M = __builtin_amdgcn_readfirstlane(a.M), N = __builtin_amdgcn_readfirstlane(a.N);
    const int ktiles = __builtin_amdgcn_readfirstlane(a.K) / KB; // stages

    // workgroup -> tile: XCD x = id % 8 owns n blocks [x * npx, (x+1) * npx), M fastest
    int mb, nb;
    tile_of_workgroup(blockIdx.x, m_blocks, n_blocks_per_xcd, &mb, &nb);
    const int m0 = mb * BM, n0 = nb * BN;
    if (n0 >= N)
        return; // uniform over the workgroup, before any barrier

    // this thread's share of the two operands of a stage (rows past the edge are clamped for loading
    // and dropped at the store)
    using StageA = OperandStage<Q, BM, NT, KB, XMODE, NEED_SX>;
    using StageB = OperandStage<P, BN, NT, KB, WMODE, NEED_SW>;
    unsigned char *lds_a = smem;
    unsigned char *lds_b = smem + BM * LDS_ROW;

    uint32_t rx0[StageA::kWords], rx1[StageA::kWords], rw0[StageB::kWords], rw1[StageB::kWords]; // next two stages
    int sum_a[StageA::kSums], sum_b[StageB::kSums];
#pragma unroll
    for (int i = 0; i < StageA::kSums; ++i)
        sum_a[i] = 0;
#pragma unroll
    for (int i = 0; i < StageB::kSums; ++i)
        sum_b[i] = 0;

    v16i acc[TM][TN];
    v16f facc[GROUPED ? TM : 1][GROUPED ? TN : 1];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0;
                if (GROUPED)
                    facc[i][j][e] = 0.f;
            }
    v16i zero16;
#pragma unroll
    for (int e = 0; e < 16; ++e)
        zero16[e] = 0;
    // GROUPED: this lane's output columns and where their scales live.  The signed route feeds
    // value * 2^(8-bits) to the MFMA: the exact power of two that undoes it rides on the scale.
    const float unshift = SIGNED ? 1.0f / (float)(1 << (16 - Q - P)) : 1.0f;
    const bool g64 = GROUPED && a.group_size == 64;
    const int groups = GROUPED ? a.K / a.group_size : 0;
    const float *wsc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
        wsc[j] = GROUPED ? a.w_scale + (size_t)min(n0 + wn * 32 * TN + j * 32 + r, N - 1) * groups : nullptr;

    // Tiles past the end are clamped to the last one instead of branching: the loop body stays one
    // basic block, so the scheduler can weave loads, unpacking and MFMAs; the duplicate tile lands
    // in the LDS buffer nobody reads again, and its row sums are masked out.
#define ABQ_LOAD_TILE(KT, RX, RW)                                                    \
    {                                                                                \
        const int kt_ld = min((KT), ktiles - 1);                                     \
        StageA::load(RX, xt, M, m0, tid, kt_ld);                                     \
        StageB::load(RW, wt, N, n0, tid, kt_ld);                                     \
    }
#define ABQ_EXPAND_TILE(RX, RW, BUF, LIVE)                                                            \
    {                                                                                                 \
        StageA::expand(RX, lds_a + (BUF) * BUF_BYTES, tid, sum_a, (LIVE));                            \
        StageB::expand(RW, lds_b + (BUF) * BUF_BYTES, tid, sum_b, (LIVE));                            \
    }

    float gsc[TN][2]; // GROUPED: scales of the stage being multiplied
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        gsc[j][0] = GROUPED ? wsc[j][0] : 0.f;
        gsc[j][1] = (GROUPED && g64) ? wsc[j][1] : gsc[j][0];
    }
    ABQ_LOAD_TILE(0, rx0, rw0)
    ABQ_LOAD_TILE(1, rx1, rw1)
    if (NEED_SX || NEED_SW)
        for (int i = tid; i < BM + BN; i += NT)
            rowsum[i] = 0;
    ABQ_EXPAND_TILE(rx0, rw0, 0, true)
    __syncthreads();

    const unsigned char *a_lane = smem + (wm * 32 * TM + r) * LDS_ROW + g * 16;
    const unsigned char *b_lane = smem + (BM + wn * 32 * TN + r) * LDS_ROW + g * 16;

    // One K tile: MFMAs on LDS buffer BUF (tile kt), loads of tile kt+2 into the register slot
    // tile kt used, expansion of tile kt+1 (other register slot) into the other LDS buffer.
#define ABQ_K_TILE(KT, BUF, RXC, RWC, RXN, RWN)                                                        \
    {                                                                                                  \
        /* the next stage's scales are requested before the tile prefetch, so that waiting for this   \
           stage's scales (requested one stage ago) never drains the prefetch behind them */          \
        float gsn[TN][2];                                                                              \
        if (GROUPED) {                                                                                 \
            const int kn = min((KT) + 1, ktiles - 1);                                                  \
            _Pragma("unroll") for (int j = 0; j < TN; ++j)                                             \
            {                                                                                          \
                gsn[j][0] = g64 ? wsc[j][2 * kn] : wsc[j][kn];                                         \
                gsn[j][1] = g64 ? wsc[j][2 * kn + 1] : gsn[j][0];                                      \
            }                                                                                          \
        }                                                                                              \
        ABQ_LOAD_TILE((KT) + 2, RXC, RWC)                                                              \
        const unsigned char *ab = a_lane + (BUF) * BUF_BYTES;                                          \
        const unsigned char *bb = b_lane + (BUF) * BUF_BYTES;                                          \
        _Pragma("unroll") for (int ks = 0; ks < WSETS; ++ks)                                           \
        {                                                                                              \
            v4i av[TM], bv[TN];                                                                        \
            _Pragma("unroll") for (int i = 0; i < TM; ++i)                                             \
                av[i] = *reinterpret_cast<const v4i *>(ab + i * 32 * LDS_ROW + ks * 32);               \
            _Pragma("unroll") for (int j = 0; j < TN; ++j)                                             \
                bv[j] = *reinterpret_cast<const v4i *>(bb + j * 32 * LDS_ROW + ks * 32);               \
            _Pragma("unroll") for (int i = 0; i < TM; ++i)                                             \
                _Pragma("unroll") for (int j = 0; j < TN; ++j)                                         \
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j],                    \
                                                                      (GROUPED && ks == 0) ? zero16 : acc[i][j], 0, 0, 0); \
            if (GROUPED && (ks == 3 || (ks == 1 && g64))) {                                            \
                _Pragma("unroll") for (int i = 0; i < TM; ++i)                                         \
                    _Pragma("unroll") for (int j = 0; j < TN; ++j)                                     \
                        _Pragma("unroll") for (int e = 0; e < 16; ++e)                                 \
                        {                                                                              \
                            facc[i][j][e] += (float)acc[i][j][e] * (gsc[j][ks >> 1] * unshift);        \
                            if (ks != WSETS - 1) /* a new stage starts from the zero operand */       \
                                acc[i][j][e] = 0;                                                      \
                        }                                                                              \
            }                                                                                          \
        }                                                                                              \
        ABQ_EXPAND_TILE(RXN, RWN, (BUF) ^ 1, (KT) + 1 < ktiles)                                        \
        if (GROUPED) {                                                                                 \
            _Pragma("unroll") for (int j = 0; j < TN; ++j)                                             \
            {                                                                                          \
                gsc[j][0] = gsn[j][0];                                                                 \
                gsc[j][1] = gsn[j][1];                                                                 \
            }                                                                                          \
        }                                                                                              \
        __syncthreads();                                                                               \
    }

    for (int kt = 0; kt < ktiles; kt += 2) {
        ABQ_K_TILE(kt, 0, rx0, rw0, rx1, rw1)
        if (kt + 1 < ktiles)
            ABQ_K_TILE(kt + 1, 1, rx1, rw1, rx0, rw0)
    }
#undef ABQ_K_TILE
#undef ABQ_EXPAND_TILE
#undef ABQ_LOAD_TILE

    if (NEED_SX || NEED_SW) {
        if (NEED_SX)
            StageA::flush_sums(rowsum, tid, sum_a);
        if (NEED_SW)
            StageB::flush_sums(rowsum + BM, tid, sum_b);
        __syncthreads();
    }

    if constexpr (GROUPED) {
        group_scale_epilogue<TM, TN, WM, WN, 2 * BUF_BYTES>(a, facc, smem, M, N, m0, n0, wm, wn, r, g, tid);
        return;
    }

    const int k_fed = ktiles * KB;
    auto result = [&](int i, int j, int e) -> int {
        unsigned v = (unsigned)acc[i][j][e];
        if (SIGNED) {
            v = (unsigned)((int)v >> (16 - Q - P));
        } else {
            if (NEED_SX)
                v += 128u * (unsigned)rowsum[wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4)];
            if (NEED_SW)
                v += 128u * (unsigned)rowsum[BM + wn * 32 * TN + j * 32 + r];
            if (NEED_SX && NEED_SW)
                v -= 16384u * (unsigned)k_fed;
        }
        return (int)v;
    };
    // fp16 outputs leave through LDS as whole lines where the output allows it (abq_group_epilogue.h); same
    // arithmetic as store_result
    using WT = WaveTileF16<TM, TN>;
    if (a.out_kind != 0 && WM * WN * WT::kBytes <= 2 * BUF_BYTES &&
        store_wave_tile_f16_ok(a.D, N, N)) {
        _Float16 *out = reinterpret_cast<_Float16 *>(a.D);
        unsigned char *region = smem + wid * WT::kBytes;
        if (a.out_kind == 2) {
            float wsv[TN], xsv[TM][16];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                wsv[j] = a.w_scale[min(n0 + wn * 32 * TN + j * 32 + r, N - 1)];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    xsv[i][e] = a.x_scale[min(m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4), M - 1)];
            __syncthreads(); // the tile buffers are free: the last K tile is behind every wave
            store_wave_tile_f16<TM, TN>(out, N, M, N, m0 + wm * 32 * TM, n0 + wn * 32 * TN, region, lane,
                                        [&](int i, int j, int e) { return (float)result(i, j, e) * xsv[i][e] * wsv[j]; });
        } else {
            const _Float16 scale = a.out_kind == 1 ? *reinterpret_cast<const _Float16 *>(a.C)
                                                   : (_Float16) * reinterpret_cast<const float *>(a.C);
            __syncthreads();
            store_wave_tile_f16<TM, TN>(out, N, M, N, m0 + wm * 32 * TM, n0 + wn * 32 * TN, region, lane,
                                        [&](int i, int j, int e) { return (float)((_Float16)(float)result(i, j, e) * scale); });
        }
        return;
    }
    const StoreOperands so = store_operands(a);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * 32 * TN + j * 32 + r;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4);
                if (m < M && n < N)
                    store_result_compact(so, m, n, result(i, j, e));
            }
        }
    }
}

template <int Q, int P, bool SIGNED, int TM, int TN, bool GROUPED, int KB, int WM = 2, int WN = 2>
static hipError_t launch_mfma_tiled(const GemmArgs &a, hipStream_t stream)
{
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    if (GROUPED && (Int8ModeOf<Q, SIGNED>::value == kFlip || Int8ModeOf<P, SIGNED>::value == kFlip))
        return hipErrorInvalidValue; // group scales with 8-bit unsigned operands: not built
    const int m_blocks = (a.M + BM - 1) / BM, n_blocks = (a.N + BN - 1) / BN;
    const int npx = (n_blocks + 7) / 8;
    const size_t lds = 2 * (size_t)(BM + BN) * (KB + 16) + (BM + BN) * sizeof(int);
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void *>(&gemm_mfma_tiled<Q, P, SIGNED, TM, TN, GROUPED, KB, WM, WN>),
        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    const dim3 grid(8 * npx * m_blocks);
    hipLaunchKernelGGL((gemm_mfma_tiled<Q, P, SIGNED, TM, TN, GROUPED, KB, WM, WN>), grid, dim3(64 * WM * WN), lds, stream, a, a.X, a.W, m_blocks, npx);
    return hipGetLastError();
}

// Native tile space of this kernel: MFMA tiles per wave (TM, TN); nstage 4 marks the K-tiled
// operand layout.  The group-scale variants sit in a table of their own and exist for the tiles
// the default choice uses.
#define ABQ_TILED_VARIANTS(V) V(4, 4) V(2, 4) V(2, 2) V(2, 1) V(1, 1)
#define ABQ_TILED_HALF_VARIANTS(V) V(2, 4) V(2, 2)   // K stage of 64
#define ABQ_TILED_WIDE_VARIANTS(V) V(2, 2, 4, 2) V(2, 2, 4, 4) V(2, 4, 4, 2)   // TM, TN, waves along M, N
#define ABQ_GROUPED_VARIANTS(V) V(2, 2) V(1, 1)

#define ABQ_ENTRY_T(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, true, TM, TN, false, 128>, 128 },
#define ABQ_ENTRY_F(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, false, TM, TN, false, 128>, 128 },
#define ABQ_HENTRY_T(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, true, TM, TN, false, 64>, 64 },
#define ABQ_HENTRY_F(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, false, TM, TN, false, 64>, 64 },
#define ABQ_WENTRY_T(TM, TN, WM, WN) { 32, TM, TN, WM, WN, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, true, TM, TN, false, 128, WM, WN>, 128 },
#define ABQ_WENTRY_F(TM, TN, WM, WN) { 32, TM, TN, WM, WN, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, false, TM, TN, false, 128, WM, WN>, 128 },
#define ABQ_GENTRY_T(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, true, TM, TN, true, 128>, 128 },
#define ABQ_GENTRY_F(TM, TN) { 32, TM, TN, 2, 2, 1, 4, &launch_mfma_tiled<ABQ_Q, ABQ_P, false, TM, TN, true, 128>, 128 },

// Pairs of single-field widths (2, 4, 8 bits) run the tiles that the staged kernel
// (abq_gemm_staged.h: records loaded straight into LDS, unpacked by the waves after the LDS read) is built
// for on that kernel, under the same tile tuples; the other tiles and pairs keep the kernel above.
#define ABQ_FIELD1(B) ((B) == 2 || (B) == 4 || (B) == 8)
#if ABQ_FIELD1(ABQ_Q) && ABQ_FIELD1(ABQ_P)
#define ABQ_SENTRY(SG, TM, TN, WM, WN)                                                       \
    { 32, TM, TN, WM, WN, 1, 4, &launch_mfma_staged<ABQ_Q, ABQ_P, SG, false, TM, TN, WM, WN>, 128, \
      StagedStages<ABQ_Q, ABQ_P, false, TM, TN, WM, WN>::kLds },
// The small tiles with two groups of waves that split K inside the workgroup (small grids).
#define ABQ_SENTRY_K(SG, TM, TN, WM, WN, WK)                                                            \
    { 32, TM, TN, WM, WN, WK, 4, &launch_mfma_staged<ABQ_Q, ABQ_P, SG, false, TM, TN, WM, WN, false, WK>, 128, \
      StagedStages<ABQ_Q, ABQ_P, false, TM, TN, WM, WN, false, WK>::kLds },
// (the 128 x 128 one where three stages of two K tiles fit the LDS: not W8A8)
#if ABQ_Q == 8 && ABQ_P == 8
#define ABQ_STAGED_KSPLIT(SG) ABQ_SENTRY_K(SG, 1, 1, 2, 2, 2) ABQ_SENTRY_K(SG, 2, 1, 2, 2, 2)
#else
#define ABQ_STAGED_KSPLIT(SG) ABQ_SENTRY_K(SG, 1, 1, 2, 2, 2) ABQ_SENTRY_K(SG, 2, 1, 2, 2, 2) ABQ_SENTRY_K(SG, 2, 2, 2, 2, 2)
#endif
// Activations wider than the weights: a 128 x 256 tile (eight waves of 64 x 64, 2 along M, 4 along N) moves fewer
// bytes per MFMA than 256 x 128, since a row of activations is the longer record.
#if ABQ_Q > ABQ_P
// ... and for small grids a 64 x 128 tile (four waves of 32 x 64), plain and with two groups of waves that split K.
#define ABQ_STAGED_WIDE_N(SG) ABQ_SENTRY(SG, 2, 2, 2, 4) ABQ_SENTRY(SG, 1, 2, 2, 2) ABQ_SENTRY_K(SG, 1, 2, 2, 2, 2)
#define ABQ_STAGED_WIDE_N_GROUPED(SG) ABQ_SGENTRY(SG, 2, 2, 2, 4) ABQ_SGENTRY(SG, 1, 2, 2, 2) ABQ_SGENTRY_K(SG, 1, 2, 2, 2, 2)
#else
#define ABQ_STAGED_WIDE_N(SG)
#define ABQ_STAGED_WIDE_N_GROUPED(SG)
#endif
// The 256 x 256 tile of eight 64 x 128 waves: on the staged kernel where three LDS stages of it fit (not W8A8).
#if ABQ_Q == 8 && ABQ_P == 8
#define ABQ_STAGED_256(SG) ABQ_WENTRY_##SG(2, 4, 4, 2)
#define ABQ_WENTRY_true(TM, TN, WM, WN) ABQ_WENTRY_T(TM, TN, WM, WN)
#define ABQ_WENTRY_false(TM, TN, WM, WN) ABQ_WENTRY_F(TM, TN, WM, WN)
#else
#define ABQ_STAGED_256(SG) ABQ_SENTRY(SG, 2, 4, 4, 2)
#endif
static const KernelEntry kSigned[] = { ABQ_ENTRY_T(4, 4) ABQ_ENTRY_T(2, 4) ABQ_SENTRY(true, 2, 2, 2, 2) ABQ_SENTRY(true, 2, 1, 2, 2)
                                       ABQ_SENTRY(true, 1, 1, 2, 2) ABQ_TILED_HALF_VARIANTS(ABQ_HENTRY_T)
                                       ABQ_SENTRY(true, 2, 2, 4, 2) ABQ_WENTRY_T(2, 2, 4, 4) ABQ_STAGED_256(true)
                                       ABQ_STAGED_WIDE_N(true) ABQ_STAGED_KSPLIT(true) };
#if ABQ_Q < 8 && ABQ_P < 8
static const KernelEntry kUnsigned[] = { ABQ_ENTRY_F(4, 4) ABQ_ENTRY_F(2, 4) ABQ_SENTRY(false, 2, 2, 2, 2) ABQ_SENTRY(false, 2, 1, 2, 2)
                                         ABQ_SENTRY(false, 1, 1, 2, 2) ABQ_TILED_HALF_VARIANTS(ABQ_HENTRY_F)
                                         ABQ_SENTRY(false, 2, 2, 4, 2) ABQ_WENTRY_F(2, 2, 4, 4) ABQ_STAGED_256(false)
                                         ABQ_STAGED_WIDE_N(false) ABQ_STAGED_KSPLIT(false) };
#else
// Pairs with an unsigned 8-bit operand: the kernel above under every tuple, which takes the row sums of the
// correction itself, and behind it, under the same tuples, the staged kernel for the tiles it is built for, which
// wants them handed in (abq_row_sums; the host launches it when it has them).
#define ABQ_SENTRY_U8(TM, TN, WM, WN)                                                           \
    { 32, TM, TN, WM, WN, 1, 4, &launch_mfma_staged<ABQ_Q, ABQ_P, false, false, TM, TN, WM, WN>, 128, \
      StagedStages<ABQ_Q, ABQ_P, false, TM, TN, WM, WN>::kLds, kNeedsRowSums },
#if ABQ_Q == 8 && ABQ_P == 8
#define ABQ_STAGED_U8_LARGE
#else
#define ABQ_STAGED_U8_LARGE ABQ_SENTRY_U8(2, 4, 4, 2)
#endif
static const KernelEntry kUnsigned[] = { ABQ_TILED_VARIANTS(ABQ_ENTRY_F) ABQ_TILED_HALF_VARIANTS(ABQ_HENTRY_F)
                                         ABQ_TILED_WIDE_VARIANTS(ABQ_WENTRY_F)
                                         ABQ_SENTRY_U8(2, 2, 2, 2) ABQ_SENTRY_U8(2, 1, 2, 2) ABQ_SENTRY_U8(1, 1, 2, 2)
                                         ABQ_SENTRY_U8(2, 2, 4, 2) ABQ_STAGED_U8_LARGE };
#endif
#else
static const KernelEntry kSigned[] = { ABQ_TILED_VARIANTS(ABQ_ENTRY_T) ABQ_TILED_HALF_VARIANTS(ABQ_HENTRY_T)
                                       ABQ_TILED_WIDE_VARIANTS(ABQ_WENTRY_T) };
static const KernelEntry kUnsigned[] = { ABQ_TILED_VARIANTS(ABQ_ENTRY_F) ABQ_TILED_HALF_VARIANTS(ABQ_HENTRY_F)
                                         ABQ_TILED_WIDE_VARIANTS(ABQ_WENTRY_F) };
#endif
// Group scales: the kernel above for groups of 64 and 128; for groups of 128 and pairs of single-field
// widths also the staged kernel (entries with a fixed LDS size), which the host prefers.
#if ABQ_FIELD1(ABQ_Q) && ABQ_FIELD1(ABQ_P)
#define ABQ_SGENTRY(SG, TM, TN, WM, WN)                                                                  \
    { 32, TM, TN, WM, WN, 1, 4, &launch_mfma_staged<ABQ_Q, ABQ_P, SG, false, TM, TN, WM, WN, true>, 128, \
      StagedStages<ABQ_Q, ABQ_P, false, TM, TN, WM, WN, true>::kLds },
// (the 128 x 64 and 128 x 128 tiles also with two groups of waves that split K, for grids of one round; the 64 x 64
// tile, one MFMA tile per wave, plain and split, for batches of 17 to 64 rows)
#define ABQ_SGENTRY_K(SG, TM, TN, WM, WN, WK)                                                                  \
    { 32, TM, TN, WM, WN, WK, 4, &launch_mfma_staged<ABQ_Q, ABQ_P, SG, false, TM, TN, WM, WN, true, WK>, 128, \
      StagedStages<ABQ_Q, ABQ_P, false, TM, TN, WM, WN, true, WK>::kLds },
#if ABQ_Q == 8 && ABQ_P == 8
// two fragment sets of 64x64 8-bit operands, the int32 and the fp32 accumulators do not fit 256 registers
#define ABQ_STAGED_GROUPED(SG) ABQ_SGENTRY(SG, 2, 1, 2, 2) ABQ_SGENTRY_K(SG, 2, 1, 2, 2, 2) ABQ_SGENTRY(SG, 1, 1, 2, 2) ABQ_SGENTRY_K(SG, 1, 1, 2, 2, 2)
#else
#define ABQ_STAGED_GROUPED(SG)                                                                                          \
    ABQ_SGENTRY(SG, 2, 2, 4, 2) ABQ_SGENTRY(SG, 2, 2, 2, 2) ABQ_SGENTRY(SG, 2, 1, 2, 2) ABQ_STAGED_WIDE_N_GROUPED(SG) \
    ABQ_SGENTRY_K(SG, 2, 1, 2, 2, 2) ABQ_SGENTRY_K(SG, 2, 2, 2, 2, 2) ABQ_SGENTRY(SG, 1, 1, 2, 2) ABQ_SGENTRY_K(SG, 1, 1, 2, 2, 2)
#endif
static const KernelEntry kSignedGrouped[] = { ABQ_GROUPED_VARIANTS(ABQ_GENTRY_T) ABQ_STAGED_GROUPED(true) };
#if ABQ_Q < 8 && ABQ_P < 8
static const KernelEntry kUnsignedGrouped[] = { ABQ_GROUPED_VARIANTS(ABQ_GENTRY_F) ABQ_STAGED_GROUPED(false) };
#else
static const KernelEntry kUnsignedGrouped[] = { ABQ_GROUPED_VARIANTS(ABQ_GENTRY_F) };
#endif
#else
static const KernelEntry kSignedGrouped[] = { ABQ_GROUPED_VARIANTS(ABQ_GENTRY_T) };
static const KernelEntry kUnsignedGrouped[] = { ABQ_GROUPED_VARIANTS(ABQ_GENTRY_F) };
#endif

#define ABQ_CAT_(a, b, c, d) a##b##c##d
#define ABQ_CAT(a, b, c, d) ABQ_CAT_(a, b, c, d)

void ABQ_CAT(abq_tiled_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSigned, (int)(sizeof(kSigned) / sizeof(kSigned[0])) };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsigned, (int)(sizeof(kUnsigned) / sizeof(kUnsigned[0])) };
}

void ABQ_CAT(abq_tiled_grouped_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSignedGrouped, (int)(sizeof(kSignedGrouped) / sizeof(kSignedGrouped[0])) };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsignedGrouped, (int)(sizeof(kUnsignedGrouped) / sizeof(kUnsignedGrouped[0])) };
}

} // namespace abq
