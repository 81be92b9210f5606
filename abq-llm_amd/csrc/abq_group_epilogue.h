// Epilogue of the prefill kernels' group-scale variants: what remains to be done once the K loop has
// folded every scale group into the fp32 accumulators.
//
//   out[m][n] = x_scale[m] * ( facc[m][n] - sum_g w_scale[n][g] * w_zero[n][g] * Sx[m][g] - x_zero[m] * T[n] )
//
// with Sx the sums of the activation codes per group and T the weight-side term of the activation zero
// points; then the optional SiLU gate and the fp16 store.    Semantics of the scales and zero points:
// algorithm/quantize/quantizer.py:111-179 of the reference.
#pragma once
#include "abq_kernels.h"

namespace abq {

typedef float v16f __attribute__((ext_vector_type(16)));

// ---- fp16 tile store through LDS ------------------------------------------------------------
// In the 32x32 accumulator layout a lane holds one column, so a direct fp16 store writes 2 bytes per
// lane, 64 bytes per row and instruction.  Going through LDS turns the wave's 32 TM x 32 TN tile
// around: every lane then stores 16 bytes (8 columns of one row), an instruction covers whole
// 128-byte lines.  Each wave uses a region of its own (wave_tile_f16_lds_bytes), so only the wave's own
// LDS traffic has to be ordered.  Needs an output row length and column count that are multiples
// of 8 and a 16-byte aligned output (store_wave_tile_f16_ok).
// CW: output columns per 32-column MFMA tile: 32, or 16 for the SiLU gate, which folds each tile's two halves
// into one: lanes r < 16 then hold the outputs of the elements e < 8 of column r, lanes r >= 16 those of the
// elements e >= 8 of column r - 16 (value(i, j, e) is only used where the lane holds an output).
template <int TM, int TN, int CW = 32> struct WaveTileF16 {
    static constexpr int kStride = 2 * CW * TN + 16;    // bytes per tile row in LDS
    static constexpr int kBytes = 32 * TM * kStride;    // per wave
    static constexpr int kLanesPerRow = CW * TN / 8;    // 16-byte chunks per row
    static constexpr int kRowsPerPass = 64 / kLanesPerRow;
};

__device__ __forceinline__ bool store_wave_tile_f16_ok(const void *out, int row_len, int cols)
{
    return (reinterpret_cast<size_t>(out) & 15) == 0 && row_len % 8 == 0 && cols % 8 == 0;
}

// value(i, j, e): element e of MFMA tile (i, j) as a float.  (row0, col0): the wave tile's origin in
// the output; rows >= rows_end and columns >= cols_end are dropped.
template <int TM, int TN, int CW = 32, typename F>
__device__ __forceinline__ void store_wave_tile_f16(_Float16 *out, int row_len, int rows_end, int cols_end, int row0, int col0,
                                                    unsigned char *wave_lds, int lane, F value)
{
    using T = WaveTileF16<TM, TN, CW>;
    const int r = lane & 31, g = lane >> 5;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const _Float16 h = (_Float16)value(i, j, e);
                if (CW == 32 || (e >> 3) == (r >> 4))
                    *reinterpret_cast<_Float16 *>(wave_lds + (i * 32 + 8 * (e / 4) + 4 * g + (e % 4)) * T::kStride +
                                                  (j * CW + (r & (CW - 1))) * 2) = h;
            }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int lr = lane / T::kLanesPerRow, lc = lane % T::kLanesPerRow;
#pragma unroll
    for (int it = 0; it < 32 * TM / T::kRowsPerPass; ++it) {
        const int row = it * T::kRowsPerPass + lr;
        typedef unsigned int line_piece __attribute__((ext_vector_type(4)));
        const line_piece v = *reinterpret_cast<const line_piece *>(wave_lds + row * T::kStride + lc * 16);
        const int m = row0 + row, n = col0 + lc * 8;
        if (m < rows_end && n < cols_end) // written once, read by another kernel: non-temporal
            __builtin_nontemporal_store(v, reinterpret_cast<line_piece *>(out + (size_t)m * row_len + n));
    }
}

typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

// Eight consecutive per-group values of one row, groups [gb, gb + 8) of `groups`, zeros past the end.  Where the
// eight exist they come as two 16-byte loads that ask for 4-byte alignment only (rows of 86 groups, K = 11008, start
// anywhere); the lanes of a last, partial chunk load one by one.
template <typename T> __device__ __forceinline__ void load_groups8(const T *row, int gb, int groups, T (&v)[8])
{
    typedef T quad __attribute__((ext_vector_type(4), aligned(4)));
    if (gb + 8 <= groups) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const quad t = *reinterpret_cast<const quad *>(row + gb + 4 * c);
#pragma unroll
            for (int d = 0; d < 4; ++d)
                v[4 * c + d] = t[d];
        }
    } else {
#pragma unroll
        for (int t = 0; t < 8; ++t)
            v[t] = gb + t < groups ? row[gb + t] : T(0);
    }
}

// Sixteen groups (from gb on) of the lane's TM activation rows and TN weight rows: group sums, scales, zero points.
template <int TM, int TN> struct ZeroPointChunk {
    int sx[2][TM][8];
    float ws[2][TN][8], wz[2][TN][8];
};

template <int TM, int TN>
__device__ __forceinline__ void zero_point_loads_half(const GemmArgs &a, const uint32_t (&arow)[TM], const uint32_t (&brow)[TN], int gb,
                                                      int groups, ZeroPointChunk<TM, TN> &c, int h)
{
#pragma unroll
    for (int i = 0; i < TM; ++i)
        load_groups8(a.x_group_sums + arow[i], gb + 8 * h, groups, c.sx[h][i]);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        load_groups8(a.w_scale + brow[j], gb + 8 * h, groups, c.ws[h][j]);
        load_groups8(a.w_zero + brow[j], gb + 8 * h, groups, c.wz[h][j]);
    }
}

template <int TM, int TN>
__device__ __forceinline__ void zero_point_loads(const GemmArgs &a, const uint32_t (&arow)[TM], const uint32_t (&brow)[TN], int gb,
                                                 int groups, ZeroPointChunk<TM, TN> &c)
{
    zero_point_loads_half<TM, TN>(a, arow, brow, gb, groups, c, 0);
    zero_point_loads_half<TM, TN>(a, arow, brow, gb, groups, c, 1);
}

// facc -= (the eight groups' sums) x (their w_scale * w_zero)^T: four bf16 MFMAs per MFMA tile, see below.
template <int TM, int TN>
__device__ __forceinline__ void zero_point_product(const int (&sx)[TM][8], const float (&ws)[TN][8], const float (&wz)[TN][8],
                                                   v16f (&facc)[TM][TN])
{
    unsigned ap[TM][8][2], bp[TN][8];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int low = sx[i][t] & 127;
            const unsigned hi = __builtin_bit_cast(unsigned, (float)(sx[i][t] - low)), lo = __builtin_bit_cast(unsigned, (float)low);
            ap[i][t][0] = __builtin_amdgcn_perm(hi, hi, 0x07060706u); // (hi, hi) as two bf16: the upper halves, exact
            ap[i][t][1] = __builtin_amdgcn_perm(lo, lo, 0x07060706u);
        }
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float c = -(ws[j][t] * wz[j][t]);
            v2bf p;
            p[0] = (__bf16)c;
            p[1] = (__bf16)(c - (float)p[0]);
            bp[j][t] = __builtin_bit_cast(unsigned, p);
        }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                // K slots of a group: (hi, hi, lo, lo) against (c1, c2, c1, c2)
                const v4u av = {ap[i][2 * q][0], ap[i][2 * q][1], ap[i][2 * q + 1][0], ap[i][2 * q + 1][1]};
                const v4u bv = {bp[j][2 * q], bp[j][2 * q], bp[j][2 * q + 1], bp[j][2 * q + 1]};
                facc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, av), __builtin_bit_cast(v8bf, bv),
                                                                     facc[i][j], 0, 0, 0);
            }
}

// A wave's 64 x 16 bytes from global memory straight into LDS at lds_addr + 16 * lane (`base` the same in every lane,
// `offset` the lane's byte offset from it).
__device__ __forceinline__ void epilogue_load_to_lds(const void *base, uint32_t offset, unsigned lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(offset),
                 "s"(base)
                 : "memory");
}

// Half h of a chunk that the workgroup has staged in LDS (see group_scale_epilogue): the lane's eight groups of its TM
// activation rows and TN weight rows.  A staged row is 128 bytes at row_at(row), its 16-byte pieces permuted by the
// row number.
template <int TM, int TN, typename RowAt>
__device__ __forceinline__ void zero_point_reads_half(RowAt row_at, int row_a, int row_s, int row_z, int g, int h,
                                                      ZeroPointChunk<TM, TN> &c)
{
    typedef int quad_i __attribute__((ext_vector_type(4)));
    typedef float quad_f __attribute__((ext_vector_type(4)));
    auto at = [&](int row, int piece) { return row_at(row) + 16 * (piece ^ ((row >> 1) & 7)); };
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int piece = 4 * g + 2 * h + p;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const quad_i v = *reinterpret_cast<const quad_i *>(at(row_a + 32 * i, piece));
#pragma unroll
            for (int d = 0; d < 4; ++d)
                c.sx[h][i][4 * p + d] = v[d];
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const quad_f s4 = *reinterpret_cast<const quad_f *>(at(row_s + 32 * j, piece));
            const quad_f z4 = *reinterpret_cast<const quad_f *>(at(row_z + 32 * j, piece));
#pragma unroll
            for (int d = 0; d < 4; ++d)
                c.ws[h][j][4 * p + d] = s4[d], c.wz[h][j][4 * p + d] = z4[d];
        }
    }
}

// Byte offset, from *base, of what a lane requests for unit u (eight rows) of a chunk staged through LDS (see
// group_scale_epilogue): rows 0 .. RA - 1 of the units are the tile's rows of group sums, then RB rows of scales, then RB
// rows of zero points; lane l brings the 16-byte piece (l % 8) ^ ((row / 2) % 8) of row 8 u + l / 8.
template <int RA, int RB>
__device__ __forceinline__ uint32_t zero_point_unit_offset(const GemmArgs &a, int u, int lane, int m0, int n0, int M, int N, int groups,
                                                           int first, const void **base)
{
    const int row = 8 * u + (lane >> 3);
    const int piece = (lane & 7) ^ ((row >> 1) & 7);
    // (a unit lies in one of the three arrays: RA and RB are multiples of 32)
    *base = 8 * u < RA ? (const void *)a.x_group_sums : 8 * u < RA + RB ? (const void *)a.w_scale : (const void *)a.w_zero;
    const int grow = row < RA ? min(m0 + row, M - 1) : min(n0 + (row < RA + RB ? row - RA : row - RA - RB), N - 1);
    // (a last, partial chunk: pieces past the row's end bring its last piece once more; the reader drops them)
    return ((uint32_t)grow * (uint32_t)groups + (uint32_t)min(first + 4 * piece, groups - 4)) * 4u;
}

__device__ __forceinline__ bool zero_point_rows_aligned(const GemmArgs &a, int groups)
{
    return (groups & 3) == 0 && ((reinterpret_cast<size_t>(a.x_group_sums) | reinterpret_cast<size_t>(a.w_scale) |
                                  reinterpret_cast<size_t>(a.w_zero)) & 15) == 0;
}

// facc[i][j][e]: MFMA tile (i, j) of this wave, element e in the 32x32 accumulator layout (row
// 8 * (e / 4) + 4 * g + e % 4, column r).  smem: the workgroup's LDS, free for reuse once a barrier has
// been passed (only the fp16 store uses it).
//
// The weight zero points are a small matrix product of their own, out -= Sx (M x groups) times
// (w_scale * w_zero)^T (groups x N), done on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16, an eighth of the
// time of the fp32 instruction per product) without loss: a group sum of at most 128 8-bit codes splits exactly
// into two bf16 numbers (its multiple of 128 and the remainder below 128), c = -w_scale * w_zero into bf16(c) and
// bf16(c - bf16(c)), both rounded to nearest, which carries c to 2^-18 relative; the four products of the pieces
// take four of the instruction's sixteen K slots, so one instruction covers four groups and a chunk of 32 groups
// takes eight per MFMA tile.  Lane (r, g) supplies row r of the activation block and column r of the weight block
// for the K slots 8 g .. 8 g + 7, i.e. for two groups; which two is free as long as both operands agree, and the
// choice here, groups 16 g + 2 q and 16 g + 2 q + 1 for instruction q of the chunk, lets every lane read its
// sixteen groups of a row as 64 contiguous bytes straight from global memory: no staging, no barrier.
// LDS_BYTES: size of the workgroup's LDS at smem.  AHEAD: how far the loads of the zero-point term run ahead of their
// use, for the kernels that have the registers: 0 = half a chunk is loaded, multiplied, then the other half (two memory
// latencies per chunk); 1 = a chunk's loads are all requested before any is used; 2 = and the next chunk's before the
// current one is multiplied (K = 11008 has three chunks).
// VIA_LDS (kernels whose K loop leaves the whole LDS free, every wave of the workgroup here): where the arrays' rows
// start on 16-byte boundaries the chunks come through LDS instead.  A lane's 16-byte pieces of 32 different rows touch 32
// cache lines per load instruction and use 32 bytes of each; with all waves of a compute unit doing that over some
// 100 KB of lines the 32 KB L1 fetches every line several times (QKV of LLaMA-7B at 16384 tokens: the term cost 10 %
// of the GEMM).  Staged, a load instruction takes eight whole rows of the workgroup's tile (every line once, no
// registers), and the lanes pick their pieces out of LDS.
// (Requesting the first chunk from inside the K loop's last trips, whose load slots and stages go to waste, was built
// and dropped: branches in the loop body, or copies of it with other requests, cost the integer tiles 40-90 spilled
// registers.)
template <int TM, int TN, int WM, int WN, int LDS_BYTES, int AHEAD = 0, bool VIA_LDS = false>
__device__ __forceinline__ void group_scale_epilogue(const GemmArgs &a, v16f (&facc)[TM][TN], unsigned char *smem, int M,
                                                     int N, int m0, int n0, int wm, int wn, int r, int g, int tid)
{
    // The rows' scales: element e of a lane sits in row 8 (e / 4) + 4 g + e % 4 of its MFMA tile, four consecutive
    // rows per e / 4.  Requested before the zero-point product, used after it.
    auto row_values = [&](const float *src, float (&v)[TM][16]) {
        const bool whole = (M & 3) == 0 && (reinterpret_cast<size_t>(src) & 15) == 0; // wave-uniform
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int mr = m0 + wm * 32 * TM + i * 32 + 8 * q + 4 * g;
                float4 s4;
                if (whole)
                    s4 = *reinterpret_cast<const float4 *>(src + min(mr, M - 4));
                else
                    s4 = make_float4(src[min(mr, M - 1)], src[min(mr + 1, M - 1)], src[min(mr + 2, M - 1)], src[min(mr + 3, M - 1)]);
                v[i][4 * q] = s4.x, v[i][4 * q + 1] = s4.y, v[i][4 * q + 2] = s4.z, v[i][4 * q + 3] = s4.w;
            }
    };
    float xs[TM][16];
    row_values(a.x_scale, xs);

    if (a.w_zero) {
        const int groups = a.K / a.group_size;
        // rows of this lane in the three arrays (32-bit element offsets: the arrays hold fewer than 2^32 elements)
        uint32_t arow[TM], brow[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
            arow[i] = (uint32_t)min(m0 + wm * 32 * TM + i * 32 + r, M - 1) * (uint32_t)groups;
#pragma unroll
        for (int j = 0; j < TN; ++j)
            brow[j] = (uint32_t)min(n0 + wn * 32 * TN + j * 32 + r, N - 1) * (uint32_t)groups;
        ZeroPointChunk<TM, TN> c0, c1;
        auto multiply = [&](const ZeroPointChunk<TM, TN> &c) {
            zero_point_product<TM, TN>(c.sx[0], c.ws[0], c.wz[0], facc);
            zero_point_product<TM, TN>(c.sx[1], c.ws[1], c.wz[1], facc);
        };
        int first = 0; // first group of the chunks still to do
        constexpr int RA = 32 * TM * WM, RB = 32 * TN * WN; // rows of the workgroup's tile
        if constexpr (VIA_LDS && (RA + 2 * RB) * 128 <= LDS_BYTES) {
            const int ra = wm * 32 * TM + r, rs = RA + wn * 32 * TN + r; // the lane's rows among the staged ones
            // (rows that start off 16-byte boundaries, K = 11008 with its 86 groups, keep the loads below: bringing them
            // through registers or four bytes a lane into the same LDS layout was no faster, and slower on the FP6 tiles)
            if (zero_point_rows_aligned(a, groups)) {
                const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
                const unsigned lds0 = (unsigned)(size_t)smem;
                // LDS: the tile's RA rows of group sums, its RB rows of scales, its RB rows of zero points, 128 bytes
                // each; a load instruction brings eight rows, the waves take them in turn
                constexpr int UNITS = (RA + 2 * RB) / 8;
                for (; first < groups; first += 32) {
                    __syncthreads(); // every wave is through with what the LDS held (the stages; the chunk before)
                    for (int u = wave; u < UNITS; u += WM * WN) { // wave-uniform
                        const void *base;
                        const uint32_t off = zero_point_unit_offset<RA, RB>(a, u, lane, m0, n0, M, N, groups, first, &base);
                        epilogue_load_to_lds(base, off, lds0 + u * 1024);
                    }
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                    auto row_at = [&](int row) { return smem + row * 128; };
                    zero_point_reads_half<TM, TN>(row_at, ra, rs, rs + RB, g, 0, c0);
                    zero_point_reads_half<TM, TN>(row_at, ra, rs, rs + RB, g, 1, c0);
                    if (first + 32 > groups) { // a partial chunk: groups past the end count nothing (their scales are some group's: finite)
#pragma unroll
                        for (int h = 0; h < 2; ++h)
#pragma unroll
                            for (int t = 0; t < 8; ++t)
                                if (first + 16 * g + 8 * h + t >= groups) {
#pragma unroll
                                    for (int i = 0; i < TM; ++i)
                                        c0.sx[h][i][t] = 0;
                                }
                    }
                    multiply(c0);
                }
            }
        }
        // (a lane's sixteen groups of chunk g0: from g0 + 16 g on)
        if constexpr (AHEAD == 2) {
            if (first < groups)
                zero_point_loads<TM, TN>(a, arow, brow, first + 16 * g, groups, c0);
            for (int g0 = first; g0 < groups; g0 += 64) {
                const bool second = g0 + 32 < groups; // wave-uniform
                if (second)
                    zero_point_loads<TM, TN>(a, arow, brow, g0 + 32 + 16 * g, groups, c1);
                multiply(c0);
                if (second) {
                    if (g0 + 64 < groups)
                        zero_point_loads<TM, TN>(a, arow, brow, g0 + 64 + 16 * g, groups, c0);
                    multiply(c1);
                }
            }
        } else if constexpr (AHEAD == 1) {
            for (int g0 = first; g0 < groups; g0 += 32) {
                zero_point_loads<TM, TN>(a, arow, brow, g0 + 16 * g, groups, c0);
                multiply(c0);
            }
        } else {
            for (int g0 = first; g0 < groups; g0 += 32) {
                zero_point_loads_half<TM, TN>(a, arow, brow, g0 + 16 * g, groups, c0, 0);
                zero_point_product<TM, TN>(c0.sx[0], c0.ws[0], c0.wz[0], facc);
                zero_point_loads_half<TM, TN>(a, arow, brow, g0 + 16 * g, groups, c0, 1);
                zero_point_product<TM, TN>(c0.sx[1], c0.ws[1], c0.wz[1], facc);
            }
        }
    }
    if (a.x_zero) {
        // the activation zero points: a rank-one term
        float xz[TM][16], wzt[TN];
        row_values(a.x_zero, xz);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            wzt[j] = a.w_zero_term[min(n0 + wn * 32 * TN + j * 32 + r, N - 1)];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    facc[i][j][e] -= xz[i][e] * wzt[j];
    }
    auto finish = [&](int i, int j, int e) -> float {
        float v = facc[i][j][e] * xs[i][e];
        if (a.act) {
            // SiLU gate: columns come in blocks of 16 gate rows followed by their 16 up rows, so the
            // partner of lane r is lane r ^ 16 of the same MFMA tile (N is a multiple of 32); lanes
            // r < 16 hold the output, column 16 * (n / 32) + n % 16 of the N / 2
            const float up = __shfl_xor(v, 16);
            v = silu(v) * up;
        }
        return v;
    };
    _Float16 *out = reinterpret_cast<_Float16 *>(a.D);
    const int wave = tid >> 6, lane = tid & 63;
    const int cols = a.act ? N / 2 : N;
    // whole lines per store where the output allows it: the wave's tile goes through a region of LDS of its own
    if (WM * WN * WaveTileF16<TM, TN, 32>::kBytes <= LDS_BYTES && store_wave_tile_f16_ok(out, cols, cols)) {
        __syncthreads(); // the LDS is free: the K loop is behind every wave
        if (a.act) {
            // SiLU gate: columns come in blocks of 16 gate rows followed by their 16 up rows, so lane r < 16 holds the
            // gate values of its 16 elements and lane r + 16 the up values of the same outputs.  The pair splits
            // the 16 outputs: one exchange of eight values each way, and either lane evaluates eight gates.
            float res[TM][TN][8];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const float lo = facc[i][j][k] * xs[i][k], hi = facc[i][j][k + 8] * xs[i][k + 8];
                        const float got = __shfl_xor(r < 16 ? hi : lo, 16);
                        res[i][j][k] = r < 16 ? silu(lo) * got : silu(got) * hi;
                    }
            store_wave_tile_f16<TM, TN, 16>(out, cols, M, cols, m0 + wm * 32 * TM, (n0 + wn * 32 * TN) / 2,
                                            smem + wave * WaveTileF16<TM, TN, 16>::kBytes, lane,
                                            [&](int i, int j, int e) { return res[i][j][e & 7]; });
        } else
            store_wave_tile_f16<TM, TN, 32>(out, cols, M, cols, m0 + wm * 32 * TM, n0 + wn * 32 * TN,
                                            smem + wave * WaveTileF16<TM, TN, 32>::kBytes, lane, finish);
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * 32 * TN + j * 32 + r;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4);
                const float v = finish(i, j, e);
                if (a.act) {
                    if (m < M && n < N && !(r & 16))
                        out[(size_t)m * (N / 2) + (n >> 5) * 16 + (n & 15)] = (_Float16)v;
                } else if (m < M && n < N) {
                    out[(size_t)m * N + n] = (_Float16)v;
                }
            }
        }
    }
}

} // namespace abq
