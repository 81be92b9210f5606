// LDS-staged GEMM core for operands that need no unpacking: the tiles go from global memory
// straight into LDS, the waves feed the matrix cores out of LDS.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for two families of operand formats:
//
//   FP6       both operands as FP6 records (abq_relayout_planes_fp6: 6-bit sign-magnitude codes, 96 bytes
//             per row and K tile of 128), v_mfma_f32_32x32x64_f8f6f4 with E2M3 x E2M3 and fp32
//             accumulation; see abq_gemm_fp6.hip for why the result is the exact integer.
//   integer   operands of 2, 4 or 8 bits in the K-tiled layout (abq_relayout_planes: one field per
//             element, 32 / 64 / 128 bytes per row and K tile), v_mfma_i32_32x32x32_i8.  The records
//             stay packed in LDS; a wave turns the field words of its own fragments into int8 with a
//             shift and a mask per four elements right before the MFMA that uses them (8-bit
//             operands need nothing).  Signed operands are placed at the top of the byte and the
//             result shifted right by 16 - q - p, unsigned ones of at most 4 bits are fed as they
//             are.  An unsigned 8-bit operand is fed as value - 128 (bit 7 flipped after the LDS read,
//             one xor per dword of the operand) and the result corrected in the epilogue with 128 x the
//             other operand's row sums, which the kernel does not take itself (gathering them beside
//             the MFMAs cost more than the staging saved): they come in through GemmArgs, computed once
//             per weight matrix and once per activation block by abq_row_sums.  The widths made of
//             several fields (3, 5, 6, 7 bits) stay on the kernel of abq_gemm_tiled.hip.
//
// global_load_lds_dwordx4 writes a wave's 64 x 16 bytes straight into LDS (at M0 + 16 * lane): no
// register staging, no ds_write instructions (LDS stores run at a third of the LDS read rate on
// this chip), and the data never crosses the vector register file.  S LDS stages: tile t + S is
// requested during tile t into the stage tile t has just left; the fragments of tile t + 1 are
// read out of LDS while the MFMAs of tile t run.  The compiler would drain every outstanding load
// of this kind before each ds_read, so they are issued from inline assembly and waited for by
// hand: every wave issues the same number of loads per tile, which makes "all but the newest n
// tiles have landed" one s_waitcnt vmcnt(n * loads per tile).  (WK > 1: a "tile" here is the K tiles of
// one trip of the K loop, one per group of waves; see the kernel's comment.)  No other vector-memory instruction
// may be in flight while that count is relied on: the kernel has none inside its K loop and
// drains the counter before its epilogue.  A register spill would be such an instruction: every
// instantiation must compile with .vgpr_spill_count 0 and no private segment (hipcc -save-temps
// shows both in the kernel's metadata), which is why the tile variants stop where they do.  One barrier per K tile.  Workgroups are numbered so
// that the 8 XCDs (workgroup id modulo 8) each work on a contiguous band of N, in groups of four m blocks
// (tile_of_workgroup).
// What bounds the kernel on LLaMA-sized problems is the rate at which L2 delivers the tiles
// (about 22 TB/s over the chip), not the matrix cores.
#pragma once
#include <type_traits>

#include "abq_group_epilogue.h"
#include "abq_kernels.h"

namespace abq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4))); // a 16-byte unit

// One operand's format: FP6 records, or BITS-wide integer fields (BITS in {2, 4, 8}).
template <int BITS, bool FP6> struct StagedOperand {
    static_assert(FP6 || BITS == 2 || BITS == 4 || BITS == 8, "single-field widths");
    static constexpr int kUnits = FP6 ? 6 : BITS;     // 16-byte units per row and K tile
    static constexpr int kRow = 16 * kUnits;          // bytes per row in LDS: the records as they are
    static constexpr int kReads = FP6 ? 3 : BITS / 2; // ds_read_b128 per lane and 32-row fragment

    // LDS placement (in bytes) of 16-byte unit `pos` = row * kUnits + unit of an operand block.  The
    // rows keep their place; units are permuted so that the fragment reads of sixteen consecutive rows
    // (same unit) hit sixteen different bank groups, while 64 consecutive units still fill 64
    // consecutive places (what one wave load delivers).  Every map is its own inverse.
    //   FP6: rows are 6 units apart; units swapped in pairs inside every second 256-byte line.
    //   integer: rows are 2, 4 or 8 units apart; the unit index is xor-ed with the number of the
    //   256-byte line (which holds 8, 4 or 2 rows), modulo the units of a row.
    static __device__ __forceinline__ int lds_offset(int pos)
    {
        return (pos ^ ((pos >> 4) & (FP6 ? 1 : kUnits - 1))) * 16;
    }
    // First unit of a row that lane half g reads as its c-th piece.  The two halves of the lanes split a
    // row's K tile in the middle; any split works as long as both operands use the same one.
    static __device__ __forceinline__ int lane_unit(int g, int c) { return kReads * g + c; }
};

// int8 MFMA operand of K step c (0..3) out of the pieces of one fragment (kReads 16-byte reads: this
// lane half's 64 elements as field words; element order as abq_bits.h: field word j of a word-set
// carries in byte c', at bits [f s, f s + f), the element at expanded dword (8 / f) j + s, byte c').
template <int BITS, bool SIGNED> __device__ __forceinline__ v4i staged_int8_operand(const v4i *piece, int c)
{
    if constexpr (BITS == 8) {
        if constexpr (SIGNED)
            return piece[c];
        else // value - 128
            return v4i{ piece[c][0] ^ (int)0x80808080u, piece[c][1] ^ (int)0x80808080u, piece[c][2] ^ (int)0x80808080u,
                        piece[c][3] ^ (int)0x80808080u };
    } else if constexpr (BITS == 4) {
        // step c <- words 2c, 2c + 1 of the lane's eight; each word holds two expanded dwords
        const uint32_t w0 = (uint32_t)piece[c / 2][2 * (c % 2)], w1 = (uint32_t)piece[c / 2][2 * (c % 2) + 1];
        if (SIGNED) // value * 16: the sign bit lands on bit 7
            return v4i{ (int)((w0 << 4) & 0xF0F0F0F0u), (int)(w0 & 0xF0F0F0F0u), (int)((w1 << 4) & 0xF0F0F0F0u),
                        (int)(w1 & 0xF0F0F0F0u) };
        return v4i{ (int)(w0 & 0x0F0F0F0Fu), (int)((w0 >> 4) & 0x0F0F0F0Fu), (int)(w1 & 0x0F0F0F0Fu),
                    (int)((w1 >> 4) & 0x0F0F0F0Fu) };
    } else {
        // step c <- word c of the lane's four; it holds four expanded dwords
        const uint32_t w = (uint32_t)piece[0][c];
        if (SIGNED) // value * 64
            return v4i{ (int)((w << 6) & 0xC0C0C0C0u), (int)((w << 4) & 0xC0C0C0C0u), (int)((w << 2) & 0xC0C0C0C0u),
                        (int)(w & 0xC0C0C0C0u) };
        return v4i{ (int)(w & 0x03030303u), (int)((w >> 2) & 0x03030303u), (int)((w >> 4) & 0x03030303u),
                    (int)((w >> 6) & 0x03030303u) };
    }
}

template <int N> __device__ __forceinline__ void staged_wait_loads()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// `base` is the same in every lane (a scalar register pair), `offset` the lane's byte offset from it.
__device__ __forceinline__ void staged_load_to_lds(const void *base, uint32_t offset, unsigned lds_addr)
{
    // the LDS address is the same in every lane; readfirstlane tells the compiler so
    // (M0 cannot be named as clobbered: the compiler reserves it, rejects it in a clobber list, and sets it up itself
    // right before each of its own uses; it keeps no value there across other instructions.)
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(offset),
                 "s"(base)
                 : "memory");
}

// The same with four bytes per lane (lane l lands at M0 + 4 * l): the group scales.
__device__ __forceinline__ void staged_load_dword_to_lds(const void *base, uint32_t offset, unsigned lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(offset),
                 "s"(base)
                 : "memory");
}

// LDS of a launch that writes fp16: the stages, or the waves' output tiles if those are larger and still fit beside
// the other workgroup of the compute unit (two for the four-wave tiles with at most four MFMA tiles a wave).
template <int TM, int TN, int WM, int WN, int STAGE_BYTES> struct StagedOutputLds {
    static constexpr int kTiles = WM * WN * WaveTileF16<TM, TN>::kBytes;
    static constexpr int kCap = ((WM * WN > 4 || TM * TN > 4) ? 160 : 80) * 1024;
    static constexpr int value = (kTiles > STAGE_BYTES && kTiles <= kCap) ? kTiles : STAGE_BYTES;
};

// QB / PB: bits of the activation / weight fields (2, 4 or 8; ignored for FP6).
//
// GROUPED: group-wise weight scales (one per 128 elements along K, i.e. per K tile: w_scale[N][K / 128]),
// per-token activation scales, optional zero points and SiLU gate, fp16 output (see abq_group_epilogue.h);
// integer fields and FP6 records alike (an FP6 tile is already fp32, its fold is one multiply-add).
// A tile's BN scales travel with its records: one more wave load or two of four bytes per lane into the
// tile's LDS stage, so they are covered by the same load counter and barrier as the records.  The int32
// accumulators cover one K tile; the MFMAs run tile by tile of the wave's TM x TN (four K steps in a
// row into the same accumulator), and while the matrix core works on one MFMA tile the vector ALU folds
// the one finished before it into the fp32 accumulators (a convert and a multiply-add per element: as
// many cycles as the four MFMAs take).  The last MFMA tile of a K tile is folded during the first of the
// next K tile.  A wave of ONE MFMA tile (the 64 x 64 workgroup tile of small batches) keeps two int32
// accumulators and alternates between them from K tile to K tile, folding the other one.
//
// WK > 1: WK groups of WM x WN waves share the workgroup's output tile and split K between them: a stage holds WK
// consecutive K tiles, group wk loads and multiplies the wk-th of them, and the groups' partial tiles meet in LDS
// after the K loop (added in a fixed order; int32 sums are exact whatever the order).  A K loop on a grid that
// leaves a compute unit one or two workgroups is a chain of latencies per K tile (wait, barrier, LDS read, four
// dependent MFMAs) that does not shrink with the tile; WK groups walk through it side by side and pay it K / (128 WK)
// times.  With a number of K tiles that is no multiple of WK the last trip finds some groups without a tile: they
// request their last tile once more, like every wave past the end, and leave its MFMAs out (with group scales: run
// them under a scale of zero).
template <int QB, int PB, bool SIGNED, bool FP6, int TM, int TN, int WM, int WN, int S, bool GROUPED = false, int WK = 1>
__global__ __launch_bounds__(64 * WM * WN * WK, (WM * WN * WK > 4 || TM * TN > 4) ? 1 : 2)
void gemm_mfma_staged(const GemmArgs a, const v4u *xt, const v4u *wt, int m_blocks, int n_blocks_per_xcd)
{
    using TA = StagedOperand<QB, FP6>;
    using TB = StagedOperand<PB, FP6>;
    constexpr int NW = WM * WN;                                // waves of one K group
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr int SC_OFF = BM * TA::kRow + BN * TB::kRow;      // GROUPED: the tile's scales follow its records
    constexpr int BUF_BYTES = SC_OFF + (GROUPED ? (BN > 128 ? 4 * BN : 512) : 0);
    constexpr int NIA = BM * TA::kUnits / 64;                  // wave loads of 1 KiB per tile: activations
    constexpr int NI = NIA + BN * TB::kUnits / 64;             // ... and in all
    constexpr int NPR = (NI + NW - 1) / NW;                    // per wave
    constexpr int NPW = NPR + (GROUPED ? 1 : 0);               // GROUPED: and one load of 64 scales (256 bytes)
    static_assert(!GROUPED || BN / 64 <= WM * WN || BN < 64, "group scales: a wave per block of 64 scales");
    constexpr int kSteps = FP6 ? 2 : 4;                        // MFMA K steps per tile of 128
    constexpr bool FLIP_X = !FP6 && !SIGNED && QB == 8, FLIP_W = !FP6 && !SIGNED && PB == 8; // fed as value - 128
    static_assert(!GROUPED || !(FLIP_X || FLIP_W), "no group scales on unsigned 8-bit operands");
    static_assert(S >= 3 && S <= 4, "three or four LDS stages");
    static_assert(NPW * S < 64, "the load counter has six bits");
    static_assert(BUF_BYTES % 512 == 0 && (BM * TA::kRow) % 512 == 0 && (32 * TA::kRow) % 256 == 0 && (32 * TB::kRow) % 256 == 0,
                  "stages, operand blocks and fragment rows keep the placement pattern");

    // fp16 outputs leave through LDS as whole lines, each wave's tile in a region of its own; where the stages are
    // smaller than that (the narrowest operand pairs), the launch asks for the larger of the two, as long as the
    // workgroups that share a compute unit still fit
    constexpr int SBUF = WK * BUF_BYTES;                       // a stage: the K tiles of all K groups
    constexpr int F16_LDS = WM * WN * WaveTileF16<TM, TN>::kBytes;
    constexpr int LDS_BYTES = StagedOutputLds<TM, TN, WM, WN, S * SBUF>::value;
    static_assert(WK == 1 || NW * TM * TN * 4096 <= S * SBUF, "the K groups' partial tiles meet in the stages");
    constexpr bool F16_VIA_LDS = F16_LDS <= LDS_BYTES;

    extern __shared__ __align__(16) unsigned char smem[]; // [S][BM rows of X | BN rows of W]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = WK > 1 ? wave / NW : 0;   // K group
    const int wid = WK > 1 ? wave % NW : wave; // wave within its K group
    const int wm = wid / WN, wn = wid % WN;
    const int r = lane & 31, g = lane >> 5;
    const int M = __builtin_amdgcn_readfirstlane(a.M), N = __builtin_amdgcn_readfirstlane(a.N);
    const int ktot = __builtin_amdgcn_readfirstlane(a.K) / 128;         // K tiles
    const int ktiles = (ktot + WK - 1) / WK;                            // trips of the K loop: a K tile per group

    int mb, nb;
    tile_of_workgroup(blockIdx.x, m_blocks, n_blocks_per_xcd, &mb, &nb);
    const int m0 = mb * BM, n0 = nb * BN;
    if (n0 >= N)
        return; // uniform over the workgroup, before any barrier

    // Wave load q of a tile fills LDS units [64 q, 64 q + 64) of the stage, activations first; the unit
    // at LDS place P of an operand block is unit lds_offset(P) / 16 of that operand's tile.  Loads past
    // the last one repeat an earlier load of the wave (same data, same place), so that every wave
    // issues NPW loads per tile.  Rows past the edge are clamped for loading and dropped at the store.
    uint32_t goff[NPW]; // bytes from the start of the operand's records of one K tile
#pragma unroll
    for (int i = 0; i < NPR; ++i) {
        int q = wid + NW * i;
        if (q >= NI)
            q -= NW;
        if (q < NIA) { // wave-uniform
            const int v = TA::lds_offset(64 * q + lane) >> 4;
            goff[i] = 16u * ((uint32_t)min(m0 + v / TA::kUnits, M - 1) * TA::kUnits + v % TA::kUnits);
        } else {
            const int v = TB::lds_offset(64 * (q - NIA) + lane) >> 4;
            goff[i] = 16u * ((uint32_t)min(n0 + v / TB::kUnits, N - 1) * TB::kUnits + v % TB::kUnits);
        }
    }
    // GROUPED: the wave's last load of a tile brings the scales of 64 weight rows (waves take the 64-row
    // blocks of the tile in turn; several waves bring the same block, which costs 256 bytes each).  The
    // offset counts bytes from the start of w_scale to the row's scale of K tile 0.
    const int sc_block = wid % (BN / 64 > 0 ? BN / 64 : 1);
    if constexpr (GROUPED)
        goff[NPR] = 4u * ((uint32_t)min(n0 + 64 * sc_block + lane, N - 1) * (uint32_t)ktot);
    const size_t stride_a = (size_t)M * TA::kUnits, stride_b = (size_t)N * TB::kUnits;
    const unsigned lds0 = (unsigned)(size_t)smem; // LDS byte address of the first stage

    using Acc = typename std::conditional<FP6, v16f, v16i>::type;
    Acc acc[TM][TN];
    Acc acc_alt[TM][TN]; // GROUPED with one MFMA tile per wave: the accumulator of the odd K tiles
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[i][j][e] = acc_alt[i][j][e] = 0;

    unsigned char *lds_a = smem + wk * BUF_BYTES; // the K group's tile within a stage
    unsigned char *lds_b = lds_a + BM * TA::kRow;
    int a_off[TA::kReads], b_off[TB::kReads];
#pragma unroll
    for (int c = 0; c < TA::kReads; ++c)
        a_off[c] = TA::lds_offset((wm * 32 * TM + r) * TA::kUnits + TA::lane_unit(g, c));
#pragma unroll
    for (int c = 0; c < TB::kReads; ++c)
        b_off[c] = TB::lds_offset((wn * 32 * TN + r) * TB::kUnits + TB::lane_unit(g, c));
    // Fragment sets as the raw 16-byte reads: the kReads pieces of activation fragment i start at
    // i * kReads, those of weight fragment j at NRA + j * kReads; the MFMA operands are cut (FP6) or
    // unpacked (integer fields) out of them when they are used.
    constexpr int NRA = TM * TA::kReads, NR = NRA + TN * TB::kReads, NM = kSteps * TM * TN;
    v4i q0[NR], q1[NR];
    auto read_piece = [&](v4i(&q)[NR], int stage, int p) {
        if (p < NRA)
            q[p] = *reinterpret_cast<const v4i *>(lds_a + stage + (p / TA::kReads) * 32 * TA::kRow + a_off[p % TA::kReads]);
        else
            q[p] = *reinterpret_cast<const v4i *>(lds_b + stage + ((p - NRA) / TB::kReads) * 32 * TB::kRow +
                                                  b_off[(p - NRA) % TB::kReads]);
    };
    auto mfma = [&](Acc &c, const v4i(&q)[NR], int i, int j, int ks, bool fresh = false) {
        const v4i *pa = &q[i * TA::kReads], *pb = &q[NRA + j * TB::kReads];
        Acc zero;
#pragma unroll
        for (int e = 0; e < 16; ++e)
            zero[e] = 0;
        if constexpr (FP6) {
            // dwords 0-5 of the 12 a lane holds are the first K step's operand, 6-11 the second's (the two
            // upper dwords of the 8-dword operand are not read for 6-bit formats)
            const v8i av = ks == 0 ? __builtin_shufflevector(pa[0], pa[1], 0, 1, 2, 3, 4, 5, -1, -1)
                                   : __builtin_shufflevector(pa[1], pa[2], 2, 3, 4, 5, 6, 7, -1, -1);
            const v8i bv = ks == 0 ? __builtin_shufflevector(pb[0], pb[1], 0, 1, 2, 3, 4, 5, -1, -1)
                                   : __builtin_shufflevector(pb[1], pb[2], 2, 3, 4, 5, 6, 7, -1, -1);
            c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, fresh ? zero : c, 2, 2, 0, 0, 0, 0);
        } else {
            c = __builtin_amdgcn_mfma_i32_32x32x32_i8(staged_int8_operand<QB, SIGNED>(pa, ks),
                                                      staged_int8_operand<PB, SIGNED>(pb, ks), fresh ? zero : c, 0, 0, 0);
        }
    };
    // The tile the next requests are for: its operands' records and its scales, all wave-uniform (scalar
    // registers), the lanes adding their 32-bit offsets.  Tiles past the end are copies of the last, into stages
    // nobody reads.
    const int first = min(wk, ktot - 1); // (a group beyond the last K tile never has one of its own)
    const v4u *xq = xt + first * stride_a, *wq = wt + first * stride_b;
    const float *sq = a.w_scale + first;
    const unsigned lds_wave = lds0 + wk * BUF_BYTES + wid * 1024;
    int kq = 0;
    auto request = [&](int stage, int i) {
        if (GROUPED && i == NPR) {
            staged_load_dword_to_lds(sq, goff[i], lds0 + wk * BUF_BYTES + stage + SC_OFF + sc_block * 256);
            return;
        }
        int q = wid + NW * i;
        if (NI % NW != 0 && q >= NI)
            q -= NW;
        // (which operand request i is for does not depend on the wave when the waves divide both operands' loads)
        const bool activations = (NIA % NW == 0 && NI % NW == 0) ? NW * i < NIA : q < NIA;
        staged_load_to_lds(activations ? (const void *)xq : (const void *)wq, goff[i], lds_wave + stage + (q - wid) * 1024);
    };
    auto next_tile = [&]() {
        if ((kq + 1) * WK + wk < ktot) {
            xq += WK * stride_a;
            wq += WK * stride_b;
            sq += WK;
        }
        ++kq;
    };

    // Tile t lives in stage t % S from its request until its fragments have been read, which happens
    // during tile t - 1; during tile t the stages therefore hold tiles t + 1 .. t + S, the last one
    // requested right then into the stage tile t has just left.
    // prologue: tiles 0 .. S-1 requested; tile 0 read into the first fragment set; tile 1 landed
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int i = 0; i < NPW; ++i)
            request(s * SBUF, i);
        next_tile();
    }
    staged_wait_loads<NPW * (S - 1)>();
    __syncthreads();
#pragma unroll
    for (int p = 0; p < NR; ++p)
        read_piece(q0, 0, p);
    // GROUPED: fp32 accumulators; scales of the K tile being multiplied (sc_cur), of the next one (sc_next)
    // and of the MFMA tile still to be folded from the previous K tile (sc_last).  The signed route feeds
    // value * 2^(8-bits) to the MFMA: the exact power of two that undoes it rides on the scale.
    v16f facc[GROUPED ? TM : 1][GROUPED ? TN : 1];
    float sc_cur[TN], sc_next[TN], sc_last = 0.f;
    const float unshift = FP6 ? 64.0f : SIGNED ? 1.0f / (float)(1 << (16 - QB - PB)) : 1.0f; // FP6: both operands carry 1/8 as their unit
    int kr = 0; // trip whose scales are read next
    auto read_scales = [&](float(&sc)[TN], int stage) {
        const float f = (WK == 1 || kr * WK + wk < ktot) ? unshift : 0.f; // a trip in which the group has no K tile
        ++kr;
#pragma unroll
        for (int j = 0; j < TN; ++j)
            sc[j] = *reinterpret_cast<const float *>(lds_a + stage + SC_OFF + (wn * 32 * TN + j * 32 + r) * 4) * f;
    };
    if constexpr (GROUPED) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    facc[i][j][e] = 0.f;
        read_scales(sc_cur, 0);
    }
    staged_wait_loads<NPW * (S - 2)>();
    __syncthreads();

    int st_req = 0;         // stage the next request goes to: the one tile t occupied
    int st_rd = SBUF;       // stage of tile t + 1
    // One K tile.  On entry every wave's share of tile KT + 1 has landed (wait + barrier at the end of
    // the previous tile), and the fragment set QC holds tile KT.  The wave's load requests and LDS reads
    // are dealt out between its MFMAs: a wave issues in order, and a burst of requests at the top of
    // the tile would hold its MFMAs back until the load unit and the LDS have taken the whole burst.
#define ABQ_STAGED_K_TILE(KT, QC, QN, LIVE)                                                                     \
    {                                                                                                           \
        _Pragma("unroll") for (int k = 0; k < NM; ++k)                                                          \
        {                                                                                                       \
            if (LIVE)                                                                                           \
                mfma(acc[(k / TN) % TM][k % TN], QC, (k / TN) % TM, k % TN, k / (TM * TN));                     \
            _Pragma("unroll") for (int d = k * NPW / NM; d < (k + 1) * NPW / NM; ++d)                           \
                request(st_req, d);                                                                             \
            _Pragma("unroll") for (int p = k * NR / NM; p < (k + 1) * NR / NM; ++p)                             \
                read_piece(QN, st_rd, p);                                                                       \
            __builtin_amdgcn_sched_barrier(0);                                                                  \
        }                                                                                                       \
        next_tile();                                                                                            \
        st_req = st_req + SBUF == S * SBUF ? 0 : st_req + SBUF;                                                 \
        st_rd = st_rd + SBUF == S * SBUF ? 0 : st_rd + SBUF;                                                    \
        staged_wait_loads<NPW * (S - 2)>(); /* tile KT + 2 has landed; the S - 2 younger ones may still fly */  \
        __syncthreads();                                                                                        \
    }

    // The same with group scales.  MFMA step k works on MFMA tile u = k / kSteps of the wave's TM x TN (K
    // step k % kSteps, the first one starting from zero); beside it the vector ALU folds its share (a
    // quarter, or half for FP6) of the tile finished before u: tile u - 1 of this K tile, or for u = 0 the last tile of the previous K tile (all
    // zeros, with a zero scale, when there is none).
#define ABQ_STAGED_K_TILE_G(KT, QC, QN, ACC, ACC_PREV)                                                          \
    {                                                                                                           \
        constexpr int NU = TM * TN;                                                                             \
        read_scales(sc_next, st_rd);                                                                            \
        _Pragma("unroll") for (int k = 0; k < NM; ++k)                                                          \
        {                                                                                                       \
            const int u = k / kSteps, ks = k % kSteps, uf = (u + NU - 1) % NU;                                  \
            mfma(ACC[u / TN][u % TN], QC, u / TN, u % TN, ks, ks == 0);                                         \
            _Pragma("unroll") for (int d = k * NPW / NM; d < (k + 1) * NPW / NM; ++d)                           \
                request(st_req, d);                                                                             \
            _Pragma("unroll") for (int p = k * NR / NM; p < (k + 1) * NR / NM; ++p)                             \
                read_piece(QN, st_rd, p);                                                                       \
            const float scf = u == 0 ? sc_last : sc_cur[uf % TN];                                               \
            _Pragma("unroll") for (int e = (16 / kSteps) * ks; e < (16 / kSteps) * (ks + 1); ++e)               \
                facc[uf / TN][uf % TN][e] += (float)ACC_PREV[uf / TN][uf % TN][e] * scf;                        \
            __builtin_amdgcn_sched_barrier(0);                                                                  \
        }                                                                                                       \
        sc_last = sc_cur[TN - 1];                                                                               \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                          \
            sc_cur[j] = sc_next[j];                                                                             \
        next_tile();                                                                                            \
        st_req = st_req + SBUF == S * SBUF ? 0 : st_req + SBUF;                                                 \
        st_rd = st_rd + SBUF == S * SBUF ? 0 : st_rd + SBUF;                                                    \
        staged_wait_loads<NPW * (S - 2)>();                                                                     \
        __syncthreads();                                                                                        \
    }

    int kt = 0;
    if constexpr (GROUPED && TM * TN == 1) {
        for (; kt + 2 <= ktiles; kt += 2) {
            ABQ_STAGED_K_TILE_G(kt, q0, q1, acc, acc_alt)
            ABQ_STAGED_K_TILE_G(kt + 1, q1, q0, acc_alt, acc)
        }
        if (kt < ktiles)
            ABQ_STAGED_K_TILE_G(kt, q0, q1, acc, acc_alt)
    } else if constexpr (GROUPED) {
        for (; kt + 2 <= ktiles; kt += 2) {
            ABQ_STAGED_K_TILE_G(kt, q0, q1, acc, acc)
            ABQ_STAGED_K_TILE_G(kt + 1, q1, q0, acc, acc)
        }
        if (kt < ktiles)
            ABQ_STAGED_K_TILE_G(kt, q0, q1, acc, acc)
    } else if constexpr (WK == 1) {
        for (; kt + 2 <= ktiles; kt += 2) {
            ABQ_STAGED_K_TILE(kt, q0, q1, true)
            ABQ_STAGED_K_TILE(kt + 1, q1, q0, true)
        }
        if (kt < ktiles)
            ABQ_STAGED_K_TILE(kt, q0, q1, true)
    } else {
        // the trips in which every group has a K tile, then the one in which only the first ktot % WK groups do
        const int full = ktot / WK;
        const bool live = full * WK + wk < ktot; // wave-uniform
        for (; kt + 2 <= full; kt += 2) {
            ABQ_STAGED_K_TILE(kt, q0, q1, true)
            ABQ_STAGED_K_TILE(kt + 1, q1, q0, true)
        }
        if (kt < full) {
            ABQ_STAGED_K_TILE(kt, q0, q1, true)
            if (full < ktiles)
                ABQ_STAGED_K_TILE(kt + 1, q1, q0, live)
        } else if (full < ktiles) {
            ABQ_STAGED_K_TILE(kt, q0, q1, live)
        }
    }
#undef ABQ_STAGED_K_TILE
#undef ABQ_STAGED_K_TILE_G
    staged_wait_loads<0>(); // the clamped requests past the last tile: nothing of ours may be in flight below

    if constexpr (GROUPED) {
        // the last MFMA tile of the last K tile is still to be folded (one tile per wave: the accumulator of that
        // K tile's parity)
        const bool in_alt = TM * TN == 1 && (ktiles & 1) == 0;
#pragma unroll
        for (int e = 0; e < 16; ++e)
            facc[TM - 1][TN - 1][e] += (float)(in_alt ? acc_alt[0][0][e] : acc[TM - 1][TN - 1][e]) * sc_last;
    }
    if constexpr (WK > 1) {
        // The K groups' partial tiles: group 1, 2, .. in turn leave theirs in LDS (lane-contiguous 16-byte pieces,
        // the place of the stages, which nobody reads any more) and group 0 adds them; the other groups are done
        // then (a barrier waits for the waves of a workgroup that have not ended).
        v4u *red = reinterpret_cast<v4u *>(smem) + (wid * TM * TN * 4) * 64 + lane;
        for (int kg = 1; kg < WK; ++kg) {
            __syncthreads();
            if (wk == kg) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            v4u v;
#pragma unroll
                            for (int c = 0; c < 4; ++c)
                                v[c] = GROUPED ? __float_as_uint(facc[GROUPED ? i : 0][GROUPED ? j : 0][4 * e + c])
                                               : (FP6 ? __float_as_uint((float)acc[i][j][4 * e + c]) : (uint32_t)acc[i][j][4 * e + c]);
                            red[((i * TN + j) * 4 + e) * 64] = v;
                        }
            }
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const v4u v = red[((i * TN + j) * 4 + e) * 64];
#pragma unroll
                            for (int c = 0; c < 4; ++c) {
                                if constexpr (GROUPED)
                                    facc[GROUPED ? i : 0][GROUPED ? j : 0][4 * e + c] += __uint_as_float(v[c]);
                                else if constexpr (FP6)
                                    acc[i][j][4 * e + c] += __uint_as_float(v[c]);
                                else
                                    acc[i][j][4 * e + c] += (int)v[c];
                            }
                        }
            }
        }
        if (wk != 0)
            return;
    }
    if constexpr (GROUPED) {
        // (the integer tiles have the registers to run the zero-point loads ahead of their use; the term's operands come
        // through LDS except on the 128 x 128 tile whose waves split K, which has no registers left for that either)
        group_scale_epilogue<TM, TN, WM, WN, LDS_BYTES, FP6 ? 0 : TM * TN == 1 ? 2 : TM * TN == 2 ? 1 : 0, WK == 1 || TM * TN < 4>(a, facc, smem, M, N, m0, n0, wm,
                                                                                                               wn, r, g, tid);
        return;
    }

    // Unsigned 8-bit operands were fed as value - 128: sum (x - 128) w = sum x w - 128 sum w, and likewise for the
    // weights; with both, 2^14 K comes on top.  The correction of a column (row) is the same for all its elements.
    // The signed W8A8 instances do the same when the host hands them row sums: then their records are those of an
    // unsigned pair written with the 128 already taken off (abq_relayout_planes_biased), and nothing was flipped here.
    constexpr bool MAY_BE_BIASED = !FP6 && SIGNED && QB == 8 && PB == 8 && !GROUPED;
    if constexpr (FLIP_X || FLIP_W || MAY_BE_BIASED) {
        const bool fix_x = FLIP_X || (MAY_BE_BIASED && a.w_row_sums != nullptr); // X was fed as value - 128
        const bool fix_w = FLIP_W || (MAY_BE_BIASED && a.x_row_sums != nullptr);
        if (fix_x || fix_w) {
            int col_fix[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                unsigned v = fix_x ? 128u * (unsigned)a.w_row_sums[min(n0 + wn * 32 * TN + j * 32 + r, N - 1)] : 0u;
                if (fix_x && fix_w)
                    v -= 16384u * (unsigned)(ktot * 128);
                col_fix[j] = (int)v;
            }
            // a lane's rows come in runs of four (e % 4): all of their sums are requested before any is used, one
            // 16-byte load per run where the run lies inside the matrix and the array allows it (one memory latency
            // for the lot: loaded one by one next to their uses they cost a latency each, 3 us on a 2048-row GEMM)
            v4i rs[TM][4];
            const bool vec_ok = (reinterpret_cast<size_t>(a.x_row_sums) & 15) == 0;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int row = m0 + wm * 32 * TM + i * 32 + 8 * b + 4 * g;
                    if (!fix_w)
                        rs[i][b] = v4i{ 0, 0, 0, 0 };
                    else if (vec_ok && row + 3 < M)
                        rs[i][b] = *reinterpret_cast<const v4i *>(a.x_row_sums + row);
                    else
                        rs[i][b] = v4i{ a.x_row_sums[min(row, M - 1)], a.x_row_sums[min(row + 1, M - 1)], a.x_row_sums[min(row + 2, M - 1)],
                                        a.x_row_sums[min(row + 3, M - 1)] };
                }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const unsigned row_fix = 128u * (unsigned)rs[i][e / 4][e % 4];
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j][e] = (int)((unsigned)acc[i][j][e] + row_fix + (unsigned)col_fix[j]);
                }
        }
    }
    auto result = [&](int i, int j, int e) -> int {
        if constexpr (FP6)
            return (int)(acc[i][j][e] * 64.0f); // both operands carry 1/8 as their unit: the sum is the result / 64, exactly
        else
            return SIGNED ? acc[i][j][e] >> (16 - QB - PB) : acc[i][j][e]; // signed fields sit at the top of their bytes
    };
    if (a.out_kind == 2) {
        // per-token x per-channel scales, fp16 out (same arithmetic as store_result): the lane's TN
        // channel scales are loaded once, a row's token scale once per row
        float wsv[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
            wsv[j] = a.w_scale[min(n0 + wn * 32 * TN + j * 32 + r, N - 1)];
        _Float16 *out = reinterpret_cast<_Float16 *>(a.D);
        using WT = WaveTileF16<TM, TN>;
        if (F16_VIA_LDS && store_wave_tile_f16_ok(out, N, N)) {
            // whole 128-byte lines per store: the wave's tile goes through a region of LDS of its own
            float xsv[TM][16];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    xsv[i][e] = a.x_scale[min(m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4), M - 1)];
            __syncthreads(); // every wave's loads have landed and its fragment reads are done: the stages are free
            store_wave_tile_f16<TM, TN>(out, N, M, N, m0 + wm * 32 * TM, n0 + wn * 32 * TN, smem + wid * WT::kBytes, lane,
                                        [&](int i, int j, int e) { return (float)result(i, j, e) * xsv[i][e] * wsv[j]; });
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4);
                const float xsv = a.x_scale[min(m, M - 1)];
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int n = n0 + wn * 32 * TN + j * 32 + r;
                    if (m < M && n < N)
                        out[(size_t)m * N + n] = (_Float16)((float)result(i, j, e) * xsv * wsv[j]);
                }
            }
        }
        return;
    }
    if (a.out_kind == 1 || a.out_kind == 3) {
        // one fp16 scale for the whole output, half(acc) * scale with both steps rounding to fp16 (the arithmetic of
        // store_result; fastertransformer/.../abqgemm/mma_any/aq_bmma_kernel.h:516-519 of the reference): through LDS
        // as whole lines where the output allows it
        _Float16 *out = reinterpret_cast<_Float16 *>(a.D);
        using WT = WaveTileF16<TM, TN>;
        if (F16_VIA_LDS && store_wave_tile_f16_ok(out, N, N)) {
            const _Float16 scale = a.out_kind == 1 ? *reinterpret_cast<const _Float16 *>(a.C)
                                                   : (_Float16) * reinterpret_cast<const float *>(a.C);
            __syncthreads(); // every wave's loads have landed and its fragment reads are done: the stages are free
            store_wave_tile_f16<TM, TN>(out, N, M, N, m0 + wm * 32 * TM, n0 + wn * 32 * TN, smem + wid * WT::kBytes, lane,
                                        [&](int i, int j, int e) { return (float)((_Float16)(float)result(i, j, e) * scale); });
            return;
        }
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

// LDS stages of a tile: as many (up to four) as leave room for the workgroups that share a compute
// unit: two for the four-wave tiles when three stages of theirs fit twice, else one.
template <int QB, int PB, bool FP6, int TM, int TN, int WM, int WN, bool GROUPED = false, int WK = 1> struct StagedStages {
    static constexpr int kBuf = WK * (32 * (TM * WM * StagedOperand<QB, FP6>::kRow + TN * WN * StagedOperand<PB, FP6>::kRow) +
                                      (GROUPED ? (32 * TN * WN > 128 ? 128 * TN * WN : 512) : 0));
    static constexpr int value = (WM * WN <= 4 && TM * TN <= 4 && 2 * 4 * kBuf > 160 * 1024 && 2 * 3 * kBuf <= 160 * 1024) ? 3
                                 : (4 * kBuf <= 160 * 1024 ? 4 : 3);
    static constexpr size_t kLds = (size_t)value * kBuf;
    static_assert(3 * kBuf <= 160 * 1024, "three stages fit a compute unit's LDS");
};

template <int QB, int PB, bool SIGNED, bool FP6, int TM, int TN, int WM, int WN, bool GROUPED = false, int WK = 1>
static hipError_t launch_mfma_staged(const GemmArgs &a, hipStream_t stream)
{
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    using Stages = StagedStages<QB, PB, FP6, TM, TN, WM, WN, GROUPED, WK>;
    constexpr int S = Stages::value;
    if (GROUPED && a.group_size != 128)
        return hipErrorInvalidValue; // one scale per K tile
    const int m_blocks = (a.M + BM - 1) / BM, n_blocks = (a.N + BN - 1) / BN;
    const int npx = (n_blocks + 7) / 8;
    const dim3 grid(8 * npx * m_blocks);
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void *>(&gemm_mfma_staged<QB, PB, SIGNED, FP6, TM, TN, WM, WN, S, GROUPED, WK>),
        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    // int32 results are stored from the registers; every other kind goes through LDS
    const size_t lds = a.out_kind == 0 ? Stages::kLds : (size_t)StagedOutputLds<TM, TN, WM, WN, (int)Stages::kLds>::value;
    hipLaunchKernelGGL((gemm_mfma_staged<QB, PB, SIGNED, FP6, TM, TN, WM, WN, S, GROUPED, WK>), grid, dim3(64 * WM * WN * WK), lds,
                       stream, a, reinterpret_cast<const v4u *>(a.X), reinterpret_cast<const v4u *>(a.W), m_blocks, npx);
    return hipGetLastError();
}

} // namespace abq
