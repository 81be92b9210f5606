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
// CW: output columns per 32-column MFMA tile: 32, or 16 when only lanes r < 16 hold an output (the SiLU
// gate folds each tile's two halves into one).
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
                const _Float16 h = (_Float16)value(i, j, e); // every lane evaluates it (it may exchange data between lanes)
                if (CW == 32 || r < CW)
                    *reinterpret_cast<_Float16 *>(wave_lds + (i * 32 + 8 * (e / 4) + 4 * g + (e % 4)) * T::kStride + (j * CW + r) * 2) = h;
            }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int lr = lane / T::kLanesPerRow, lc = lane % T::kLanesPerRow;
#pragma unroll
    for (int it = 0; it < 32 * TM / T::kRowsPerPass; ++it) {
        const int row = it * T::kRowsPerPass + lr;
        const uint4 v = *reinterpret_cast<const uint4 *>(wave_lds + row * T::kStride + lc * 16);
        const int m = row0 + row, n = col0 + lc * 8;
        if (m < rows_end && n < cols_end)
            *reinterpret_cast<uint4 *>(out + (size_t)m * row_len + n) = v;
    }
}

constexpr int kZeroPointChunk = 32;                      // groups staged through LDS at a time
constexpr int kZeroPointRow = kZeroPointChunk + 1;       // floats per staged row: odd, so that 32 rows hit 32 banks

// LDS the zero-point staging needs for a BM x BN tile.
constexpr int zero_point_lds_bytes(int bm, int bn) { return (bm + bn) * kZeroPointRow * 4; }

// facc[i][j][e]: MFMA tile (i, j) of this wave, element e in the 32x32 accumulator layout (row
// 8 * (e / 4) + 4 * g + e % 4, column r).  smem: the workgroup's LDS, free for reuse once a barrier has
// been passed; zero_point_lds_bytes(BM, BN) of it are used when w_zero is set.
//
// The weight zero points are a small matrix product of their own, out -= Sx (M x groups) times
// (w_scale * w_zero)^T (groups x N).  Both factors are staged through LDS 32 groups at a time (coalesced
// loads along the groups) and multiplied on the fp32 matrix cores: v_mfma_f32_32x32x2_f32, lane (r, g)
// supplies row r of the activation block and column r of the weight block for the g-th of the
// instruction's two K indices.
// LDS_BYTES: size of the workgroup's LDS at smem.
template <int TM, int TN, int WM, int WN, int LDS_BYTES>
__device__ __forceinline__ void group_scale_epilogue(const GemmArgs &a, v16f (&facc)[TM][TN], unsigned char *smem, int M,
                                                     int N, int m0, int n0, int wm, int wn, int r, int g, int tid)
{
    static_assert(zero_point_lds_bytes(32 * TM * WM, 32 * TN * WN) <= LDS_BYTES, "the zero-point staging fits");
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr int GC = kZeroPointChunk, GP = kZeroPointRow;
    if (a.w_zero) {
        const int groups = a.K / a.group_size;
        float *zs_x = reinterpret_cast<float *>(smem); // [BM][GP]
        float *zs_w = zs_x + BM * GP;                  // [BN][GP], negated
        for (int g0 = 0; g0 < groups; g0 += GC) {
            __syncthreads();
            // every thread's loads of a chunk are issued back to back (trip counts are compile-time)
            static_assert((GC * BM) % NT == 0 && (GC * BN) % NT == 0, "whole passes of the workgroup");
            float vx[GC * BM / NT], vw[GC * BN / NT];
#pragma unroll
            for (int it = 0; it < GC * BM / NT; ++it) {
                const int u = tid + it * NT, rr = u / GC, gl = u % GC;
                const int m = min(m0 + rr, M - 1);
                vx[it] = g0 + gl < groups ? (float)a.x_group_sums[(size_t)m * groups + g0 + gl] : 0.f;
            }
#pragma unroll
            for (int it = 0; it < GC * BN / NT; ++it) {
                const int u = tid + it * NT, rr = u / GC, gl = u % GC;
                const size_t idx = (size_t)min(n0 + rr, N - 1) * groups + g0 + gl;
                vw[it] = g0 + gl < groups ? -(a.w_scale[idx] * a.w_zero[idx]) : 0.f;
            }
#pragma unroll
            for (int it = 0; it < GC * BM / NT; ++it) {
                const int u = tid + it * NT;
                zs_x[(u / GC) * GP + u % GC] = vx[it];
            }
#pragma unroll
            for (int it = 0; it < GC * BN / NT; ++it) {
                const int u = tid + it * NT;
                zs_w[(u / GC) * GP + u % GC] = vw[it];
            }
            __syncthreads();
            const float *xa = zs_x + (wm * 32 * TM + r) * GP + g;
            const float *wb = zs_w + (wn * 32 * TN + r) * GP + g;
#pragma unroll 4
            for (int t = 0; t < GC / 2; ++t) {
                float av[TM], bv[TN];
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    av[i] = xa[i * 32 * GP + 2 * t];
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    bv[j] = wb[j * 32 * GP + 2 * t];
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        facc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], facc[i][j], 0, 0, 0);
            }
        }
    }
    // what is left per element: the activation zero points (a rank-one term), the token scale, the gate
    auto finish = [&](int i, int j, int e) -> float {
        const int mc = min(m0 + wm * 32 * TM + i * 32 + 8 * (e / 4) + 4 * g + (e % 4), M - 1);
        const int nc = min(n0 + wn * 32 * TN + j * 32 + r, N - 1);
        float v = facc[i][j][e];
        if (a.x_zero)
            v -= a.x_zero[mc] * a.w_zero_term[nc];
        v *= a.x_scale[mc];
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
        __syncthreads(); // the LDS is free: K loop and zero-point staging are behind every wave
        if (a.act)
            store_wave_tile_f16<TM, TN, 16>(out, cols, M, cols, m0 + wm * 32 * TM, (n0 + wn * 32 * TN) / 2,
                                            smem + wave * WaveTileF16<TM, TN, 16>::kBytes, lane, finish);
        else
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
