// GEMM core for decode-sized M (at most 16 activation rows per grid row): matrix-core strategy
// with the activations expanded once per workgroup.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for one (x_bits, w_bits) pair per
// translation unit: compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>.
//
// The weights are the only large operand: every weight word is read exactly once, with 16-byte
// loads straight from the reference layout, by the lane that expands it to int8 and feeds it to
// v_mfma_i32_16x16x64_i8 as the B operand (no LDS round trip for weights).
// The activations are a few KiB.  Expanding them per wave costs more VALU time than the whole
// weight stream takes from HBM, so the workgroup expands them once into LDS
// (xs[row][K bytes], the byte order the expansion routine produces) and every wave reads its A
// operands from there with ds_read_b128.
//
// Work split.  The grid is persistent: at most one workgroup per compute unit, workgroup b owns
// the 16-row weight tiles b, b+G, b+2G, ...  Inside a workgroup the work items are
// (tile, K step) pairs, a step being 16 plane words (512 K elements) per row; wave w takes
// items w, w+NW, ...  Partial 16x16 results meet in LDS with ds_add (integer, so the order does
// not matter) and are written out once at the end.  K is processed in chunks sized so that the
// expanded activations fit the LDS budget; one chunk covers all baseline shapes up to M = 8.
#include "abq_kernels.h"

#ifndef ABQ_Q
#error "compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>"
#endif

namespace abq {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kDecodeMaxTiles = 8;            // weight tiles per workgroup
constexpr int kDecodeXBudget = 128 * 1024;    // bytes of LDS for the expanded activations
constexpr int kDecodeFixedLds = kDecodeMaxTiles * (256 + 16) * 4 + 16 * 4;

__device__ __forceinline__ uint32_t comp4(const uint4 &v, int i)
{
    return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

// Loads the P x SW plane words [word, word+SW) of weight row (tile*16 + r), SW = 4 (16 bytes) or 2;
// all-zero when the item or the words are out of range (one predicated region for all planes).
template <int P, int SW = 4>
__device__ __forceinline__ void load_weight_words(uint4 (&dst)[P], const uint32_t *W, size_t wplane, int KW,
                                                  int N, int tile, int r, int word, int word_end, bool item_valid)
{
#pragma unroll
    for (int b = 0; b < P; ++b)
        dst[b] = make_uint4(0u, 0u, 0u, 0u);
    if (item_valid && word < word_end) {
        const uint32_t *p = W + (size_t)min(tile * 16 + r, N - 1) * KW + word;
#pragma unroll
        for (int b = 0; b < P; ++b) {
            if (SW == 4) {
                dst[b] = *reinterpret_cast<const uint4 *>(p);
            } else {
                const uint2 v = *reinterpret_cast<const uint2 *>(p);
                dst[b].x = v.x;
                dst[b].y = v.y;
            }
            p += wplane;
        }
    }
}

// Expands the SW plane words per plane held in wv into the 2 * SW B operands of one K step.
template <int P, Int8Mode MODE, bool SUM, int SW = 4>
__device__ __forceinline__ void expand_weight_words(const uint4 (&wv)[P], v4i (&bops)[2 * SW], int &value_sum)
{
    value_sum = 0;
#pragma unroll
    for (int ws = 0; ws < SW; ++ws) {
        uint32_t w[P], bop[8];
#pragma unroll
        for (int b = 0; b < P; ++b)
            w[b] = comp4(wv[b], ws);
        if (SUM)
            value_sum += planes_value_sum<P>(w);
        planes_to_int8<P, MODE>(w, bop);
        bops[ws * 2] = v4i{ (int)bop[0], (int)bop[1], (int)bop[2], (int)bop[3] };
        bops[ws * 2 + 1] = v4i{ (int)bop[4], (int)bop[5], (int)bop[6], (int)bop[7] };
    }
}

// SW: plane words per lane and item, 4 (a step is 16 words = 512 K elements, 16-byte loads) or 2
// (steps of 256 elements: twice as many, half as long items, which spreads short K over all waves).
template <int Q, int P, bool SIGNED, int NW, int SW>
__global__ __launch_bounds__(64 * NW) void gemm_mfma_decode(const GemmArgs a, int chunk_words, int row_words,
                                                            int tw_base, int tw_rem)
{
    constexpr int NT = 64 * NW;
    constexpr int STEPW = 4 * SW;      // plane words per row and step
    constexpr int STEPB = 32 * STEPW;  // bytes of expanded activations per row and step
    constexpr Int8Mode XMODE = Int8ModeOf<Q, SIGNED>::value;
    constexpr Int8Mode WMODE = Int8ModeOf<P, SIGNED>::value;
    constexpr bool NEED_SX = WMODE == kFlip; // see abq_gemm_mfma.hip: row-sum corrections for
    constexpr bool NEED_SW = XMODE == kFlip; // 8-bit unsigned operands fed as value - 128

    extern __shared__ __align__(16) unsigned char smem[];
    int *tacc = reinterpret_cast<int *>(smem);                 // [kDecodeMaxTiles][16][16]
    int *tsw = tacc + kDecodeMaxTiles * 256;                   // [kDecodeMaxTiles][16]
    int *sxs = tsw + kDecodeMaxTiles * 16;                     // [16]
    unsigned char *xs = smem + kDecodeFixedLds;                // [Mb][RS]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // wave-uniform: everything derived from it (item -> tile / step) runs on the scalar unit
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15;
    const int g = lane >> 4;
    const int M = a.M, N = a.N, KW = a.KW;
    const int m0 = blockIdx.y * 16;
    const int Mb = min(16, M - m0);
    const int RS = row_words * 32 + 16; // row stride of xs in bytes (row_words = chunk rounded up to a step)
    const size_t xplane = (size_t)M * KW;
    const size_t wplane = (size_t)N * KW;
    const int G = gridDim.x;
    const int TW = tw_base + ((int)blockIdx.x < tw_rem ? 1 : 0); // tiles b, b+G, ... of this workgroup

    // Work items of this wave: j = wid, wid+NW, ... over (tile, step) pairs of the chunk, step
    // fastest.  (tl, st) is the item being computed, (tl1, st1) the next one.
    uint4 w1[P], w2[P];     // raw weight words of the next item and of the one after it
    uint32_t xcur[Q], xnext[Q];
    v4i bops[2 * SW];       // expanded weights of the item being computed
    int bsum = 0;
    int tl = 0, st = wid, tl1, st1;

    // Load order at entry: first the activation words this wave will expand (a few KiB in all,
    // but the expansion, the LDS write and a barrier hang off them, so they must not queue
    // behind the weight stream), then the weight words of the wave's first two items.
    // Everything up to the first MFMA overlaps the weight latency.  The scheduling barrier keeps
    // the compiler from hoisting loop-invariant setup in front of the loads.
    {
        const int cw = min(chunk_words, KW);
        const int bpr = (cw + 63) >> 6;
        int m = 0, kb = wid;
        while (kb >= bpr) {
            kb -= bpr;
            ++m;
        }
        const int kw = kb * 64 + lane;
#pragma unroll
        for (int b = 0; b < Q; ++b)
            xcur[b] = 0u;
        if (m < Mb && kw < cw) {
            const uint32_t *xp = a.X + (size_t)(m0 + m) * KW + kw;
#pragma unroll
            for (int b = 0; b < Q; ++b) {
                xcur[b] = *xp;
                xp += xplane;
            }
        }
        const int csteps = (cw + STEPW - 1) / STEPW;
        while (st >= csteps) {
            st -= csteps;
            ++tl;
        }
        st1 = st + NW;
        tl1 = tl;
        while (st1 >= csteps) {
            st1 -= csteps;
            ++tl1;
        }
        uint4 w0[P];
        load_weight_words<P, SW>(w0, a.W, wplane, KW, N, blockIdx.x + tl * G, r, st * STEPW + SW * g, cw, tl < TW);
        load_weight_words<P, SW>(w1, a.W, wplane, KW, N, blockIdx.x + tl1 * G, r, st1 * STEPW + SW * g, cw, tl1 < TW);
        __builtin_amdgcn_sched_barrier(0);
        for (int i = tid; i < kDecodeMaxTiles * (256 + 16) + 16; i += NT)
            tacc[i] = 0; // ordered before the first ds_add by the barrier that ends the expansion
        if (NEED_SX)
            __syncthreads(); // the activation row sums are accumulated during the expansion itself
        // The first item's weights are expanded while other waves expand activations.
        if (Mb * bpr <= wid)
            expand_weight_words<P, WMODE, NEED_SW, SW>(w0, bops, bsum);
        else {
#pragma unroll
            for (int b = 0; b < P; ++b)
                w2[b] = w0[b]; // this wave expands activations first; weights right after
        }
    }

    int k_fed = 0;
    for (int c0 = 0; c0 < KW; c0 += chunk_words) {
        const int cw = min(chunk_words, KW - c0);
        const int csteps = (cw + STEPW - 1) / STEPW;
        const int bpr = (cw + 63) >> 6;
        const int wend = c0 + cw;
        k_fed += csteps * STEPW * 32;
        const bool has_x_work = wid < Mb * bpr;

        if (c0 != 0) { // later chunks (long K with many activation rows): same first loads, in place
            const int m = wid / bpr;
            const int kw = (wid - m * bpr) * 64 + lane;
#pragma unroll
            for (int b = 0; b < Q; ++b)
                xcur[b] = 0u;
            if (m < Mb && kw < cw) {
                const uint32_t *xp = a.X + (size_t)(m0 + m) * KW + c0 + kw;
#pragma unroll
                for (int b = 0; b < Q; ++b) {
                    xcur[b] = *xp;
                    xp += xplane;
                }
            }
            tl = wid / csteps;
            st = wid - tl * csteps;
            st1 = st + NW;
            tl1 = tl;
            while (st1 >= csteps) {
                st1 -= csteps;
                ++tl1;
            }
            load_weight_words<P, SW>(w2, a.W, wplane, KW, N, blockIdx.x + tl * G, r, c0 + st * STEPW + SW * g, wend, tl < TW);
            load_weight_words<P, SW>(w1, a.W, wplane, KW, N, blockIdx.x + tl1 * G, r, c0 + st1 * STEPW + SW * g, wend, tl1 < TW);
            __syncthreads(); // previous chunk fully consumed before xs is overwritten
            if (!has_x_work)
                expand_weight_words<P, WMODE, NEED_SW, SW>(w2, bops, bsum);
        }

        // Activation expansion: wave-sized blocks of 64 consecutive plane words of one row,
        // the words of the next block in flight while this one is expanded.
        for (int blk = wid; blk < Mb * bpr; blk += NW) {
            const int m = blk / bpr;
            const int kw = (blk - m * bpr) * 64 + lane;
            {
                const int bn = blk + NW;
                const int mn = bn / bpr;
                const int kwn = (bn - mn * bpr) * 64 + lane;
#pragma unroll
                for (int b = 0; b < Q; ++b)
                    xnext[b] = 0u;
                if (mn < Mb && kwn < cw) {
                    const uint32_t *xp = a.X + (size_t)(m0 + mn) * KW + c0 + kwn;
#pragma unroll
                    for (int b = 0; b < Q; ++b) {
                        xnext[b] = *xp;
                        xp += xplane;
                    }
                }
            }
            if (kw < cw) {
                uint32_t o[8];
                if (NEED_SX)
                    atomicAdd(&sxs[m], planes_value_sum<Q>(xcur));
                planes_to_int8<Q, XMODE>(xcur, o);
                uint4 *dst = reinterpret_cast<uint4 *>(xs + (size_t)m * RS + kw * 32);
                dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
                dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
            }
#pragma unroll
            for (int b = 0; b < Q; ++b)
                xcur[b] = xnext[b];
        }
        // The tail of a partial last step must hold what all-zero planes expand to (weights
        // past K are fed as zero planes; the row-sum correction counts these elements).
        if (cw % STEPW) {
            const int pad = csteps * STEPW - cw;
            const uint32_t fill = XMODE == kFlip ? 0x80808080u : 0u;
            for (int u = tid; u < Mb * pad * 2; u += NT) {
                const int m = u / (pad * 2), q16 = u - m * (pad * 2);
                reinterpret_cast<uint4 *>(xs + (size_t)m * RS + cw * 32)[q16] = make_uint4(fill, fill, fill, fill);
            }
        }
        if (has_x_work)
            expand_weight_words<P, WMODE, NEED_SW, SW>(w2, bops, bsum);
        __syncthreads();

        v4i acc = { 0, 0, 0, 0 };
        int sw_part = 0;
        int cur_tl = tl < TW ? tl : -1;
        const unsigned char *xrow = xs + (size_t)min(r, Mb - 1) * RS + g * (32 * SW);

        while (tl < TW) {
            // A operands of this step: 2 * SW x 16 bytes per lane
            v4i aop[2 * SW];
            {
                const unsigned char *xw = xrow + st * STEPB;
#pragma unroll
                for (int i = 0; i < 2 * SW; ++i)
                    aop[i] = *reinterpret_cast<const v4i *>(xw + i * 16);
            }
            // weights of the item after next go in flight now
            int st2 = st1 + NW, tl2 = tl1;
            while (st2 >= csteps) {
                st2 -= csteps;
                ++tl2;
            }
            load_weight_words<P, SW>(w2, a.W, wplane, KW, N, blockIdx.x + tl2 * G, r, c0 + st2 * STEPW + SW * g, wend, tl2 < TW);
            if (tl != cur_tl) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (4 * g + e < Mb)
                        atomicAdd(&tacc[cur_tl * 256 + (4 * g + e) * 16 + r], acc[e]);
                if (NEED_SW)
                    atomicAdd(&tsw[cur_tl * 16 + r], sw_part);
                acc = v4i{ 0, 0, 0, 0 };
                sw_part = 0;
                cur_tl = tl;
            }
            sw_part += bsum;
#pragma unroll
            for (int i = 0; i < 2 * SW; ++i)
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[i], bops[i], acc, 0, 0, 0);
            // expand the next item's weights (loaded one iteration ago) for the next round
            if (tl1 < TW)
                expand_weight_words<P, WMODE, NEED_SW, SW>(w1, bops, bsum);
#pragma unroll
            for (int b = 0; b < P; ++b)
                w1[b] = w2[b];
            st = st1;
            tl = tl1;
            st1 = st2;
            tl1 = tl2;
        }
        if (cur_tl >= 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (4 * g + e < Mb)
                    atomicAdd(&tacc[cur_tl * 256 + (4 * g + e) * 16 + r], acc[e]);
            if (NEED_SW)
                atomicAdd(&tsw[cur_tl * 16 + r], sw_part);
        }
    }
    __syncthreads();

    // Output: 16 lanes per row of a tile; thread (s = tid / 16, c = tid % 16) serves row s % 16 of
    // tiles s / 16, s / 16 + NT / 256, ...
    {
        const int c = tid & 15, i = (tid >> 4) & 15;
        for (int t = tid >> 8; t < TW; t += NT / 256) {
            const int n = (blockIdx.x + t * G) * 16 + c;
            if (i < Mb && n < N) {
                unsigned v = (unsigned)tacc[t * 256 + i * 16 + c];
                if (SIGNED) {
                    v = (unsigned)((int)v >> (16 - Q - P));
                } else {
                    if (NEED_SX)
                        v += 128u * (unsigned)sxs[i];
                    if (NEED_SW)
                        v += 128u * (unsigned)tsw[t * 16 + c];
                    if (NEED_SX && NEED_SW)
                        v -= 16384u * (unsigned)k_fed;
                }
                store_result(a, m0 + i, n, (int)v);
            }
        }
    }
}

// K chunking: the whole K in one chunk if the expanded activations fit the LDS budget, else
// the largest multiple of 16 plane words that does.  row_words is the chunk rounded up to a
// whole step (16 words), the length each LDS row is laid out for.
static void decode_chunking(int M, int KW, int *chunk_words, int *row_words)
{
    const int mb = M < 16 ? M : 16;
    const int kwp = (KW + 15) / 16 * 16;
    if ((long)mb * (kwp * 32 + 16) <= kDecodeXBudget) {
        *chunk_words = KW;
        *row_words = kwp;
        return;
    }
    int cw = (kDecodeXBudget / mb - 16) / 32;
    cw -= cw % 16;
    *chunk_words = cw;
    *row_words = cw;
}

template <int Q, int P, bool SIGNED, int NW, int SW>
static hipError_t launch_mfma_decode(const GemmArgs &a, hipStream_t stream)
{
    const int tiles = (a.N + 15) / 16;
    int gx = tiles < 256 ? tiles : 256; // one workgroup per MI355X compute unit
    if ((tiles + gx - 1) / gx > kDecodeMaxTiles)
        gx = (tiles + kDecodeMaxTiles - 1) / kDecodeMaxTiles;
    int cw, rw;
    decode_chunking(a.M, a.KW, &cw, &rw);
    const int mb = a.M < 16 ? a.M : 16;
    const size_t lds = kDecodeFixedLds + (size_t)mb * (rw * 32 + 16);
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void *>(&gemm_mfma_decode<Q, P, SIGNED, NW, SW>),
        hipFuncAttributeMaxDynamicSharedMemorySize, kDecodeFixedLds + kDecodeXBudget);
    if (attr != hipSuccess)
        return attr;
    const dim3 grid(gx, (a.M + 15) / 16);
    hipLaunchKernelGGL((gemm_mfma_decode<Q, P, SIGNED, NW, SW>), grid, dim3(64 * NW), lds, stream, a, cw, rw, tiles / gx, tiles % gx);
    return hipGetLastError();
}

// ---- decode with group-wise weight scales ----------------------------------------------------
//
// D[m][n] = x_scale[m] * ( sum_g w_scale[n][g] * (acc_g - w_zero[n][g] * Sx[m][g]) - x_zero[m] * T[n] ),
// acc_g the integer dot product over scale group g (64 or 128 elements along K); semantics of
// algorithm/quantize/quantizer.py:111-179 of the reference, fp16 output.
//
// Same plan as above: activations expanded once per workgroup into LDS, weights read once with
// 16-byte loads and fed to v_mfma_i32_16x16x64_i8 as the B operand, work items = (tile, 512-K
// step).  In a step lane group g = lane / 16 holds the 128-element block 4*step + g of its weight
// row, and an MFMA sums over the four lane groups, i.e. over four scale groups.  To keep them
// apart the step is run four times with the A operand of all but one lane group read from a
// page of zeros: 32 MFMAs per step instead of 8, which a bandwidth-bound kernel can afford.
// For groups of 64 the two halves of a block (plane words 0-1 and 2-3) go to separate
// accumulators.  The block sums are folded into fp32 with their scales; the waves' partial
// tiles meet in LDS in a fixed order (deterministic sums), tiles_per_pass tiles at a time.
template <int Q, int P, bool SIGNED>
__global__ __launch_bounds__(64 * kDecodeGroupedWaves) void gemm_decode_grouped(const GemmArgs a, int tiles_per_wg,
                                                                                int tiles_per_pass)
{
    constexpr int NW = kDecodeGroupedWaves, NT = 64 * NW;
    constexpr Int8Mode XMODE = Int8ModeOf<Q, SIGNED>::value;
    constexpr Int8Mode WMODE = Int8ModeOf<P, SIGNED>::value;

    extern __shared__ __align__(16) unsigned char smem[];
    float *part = reinterpret_cast<float *>(smem);              // [tiles_per_pass][NW][16][16] per-wave partial tiles
    float *sxg = part + tiles_per_pass * NW * 256;              // [16][groups] activation group sums
    const int M = a.M, N = a.N, KW = a.KW;
    const int groups = a.K / a.group_size;
    const bool g64 = a.group_size == 64;
    const int blocks = KW / 4;                                  // 128-element blocks of K
    const int steps = (KW + 15) >> 4;                           // 512-element steps, the last one may be partial
    unsigned char *zero_page = reinterpret_cast<unsigned char *>(sxg + 16 * groups); // 128 bytes
    unsigned char *xs = zero_page + 128;                        // [Mb][RS]
    const int RS = steps * 512 + 16;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.y * 16;
    const int Mb = min(16, M - m0);
    const size_t xplane = (size_t)M * KW, wplane = (size_t)N * KW;
    const int ntiles = (N + 15) / 16;
    const int G = gridDim.x;
    // Tiles of this workgroup: blockIdx.x, blockIdx.x + G, ...; with the SiLU gate the unit is a pair of
    // tiles (16 gate rows and their 16 up rows), so that both halves of an output meet in one workgroup.
    const int unit = a.act ? 2 : 1;
    const int nunits = ntiles / unit;
    const int TW = min(tiles_per_wg, unit * ((nunits - (int)blockIdx.x + G - 1) / G));
    auto tile_of = [&](int tl) { return unit == 2 ? 2 * ((int)blockIdx.x + (tl >> 1) * G) + (tl & 1) : (int)blockIdx.x + tl * G; };

    // Work items: (tile, step) pairs, step fastest; wave w takes items w, w + NW, ... of a pass.
    // The first item's weight words go in flight before the activation work.
    uint4 wnext[P];
    {
        const int tp0 = min(tiles_per_pass, TW);
        const int tl = wid / steps, st = wid - tl * steps;
        load_weight_words<P>(wnext, a.W, wplane, KW, N, tile_of(tl), r, st * 16 + 4 * g, KW, wid < tp0 * steps);
    }

    // activations -> int8 in LDS, one wave per 64 plane words of a row; the tail of a partial last
    // step and the zero page are cleared
    {
        const int bpr = (KW + 63) >> 6;
        for (int blk = wid; blk < Mb * bpr; blk += NW) {
            const int m = blk / bpr;
            const int kw = (blk - m * bpr) * 64 + lane;
            if (kw < KW) {
                uint32_t xw[Q], o[8];
                const uint32_t *xp = a.X + (size_t)(m0 + m) * KW + kw;
#pragma unroll
                for (int b = 0; b < Q; ++b) {
                    xw[b] = *xp;
                    xp += xplane;
                }
                planes_to_int8<Q, XMODE>(xw, o);
                uint4 *dst = reinterpret_cast<uint4 *>(xs + (size_t)m * RS + kw * 32);
                dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
                dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
            }
        }
        const int pad = steps * 16 - KW; // plane words
        for (int u = tid; u < Mb * pad * 2; u += NT) {
            const int m = u / (pad * 2), q16 = u - m * (pad * 2);
            reinterpret_cast<uint4 *>(xs + (size_t)m * RS + KW * 32)[q16] = make_uint4(0u, 0u, 0u, 0u);
        }
        if (tid < 8)
            reinterpret_cast<uint4 *>(zero_page)[tid] = make_uint4(0u, 0u, 0u, 0u);
        for (int i = tid; i < 16 * groups; i += NT) {
            const int m = i / groups;
            sxg[i] = (a.w_zero && m < Mb) ? (float)a.x_group_sums[(size_t)(m0 + m) * groups + (i - m * groups)] : 0.f;
        }
    }
    __syncthreads();

    // the signed route feeds value * 2^(8-bits): the exact power of two that undoes it rides on the scale
    const float unshift = SIGNED ? 1.0f / (float)(1 << (16 - Q - P)) : 1.0f;
    const unsigned char *xrow = xs + (size_t)min(r, Mb - 1) * RS + g * 128;

    for (int t0 = 0; t0 < TW; t0 += tiles_per_pass) {
        const int tp = min(tiles_per_pass, TW - t0);
        const int items = tp * steps;
        // this wave's slots start at zero: it writes only the tiles it has items of
        for (int i = lane; i < tp * 256; i += 64)
            part[((i >> 8) * NW + wid) * 256 + (i & 255)] = 0.f;

        float facc[4] = { 0.f, 0.f, 0.f, 0.f };
        int cur_tl = -1;
        for (int j = wid; j < items; j += NW) {
            const int tl = j / steps, st = j - tl * steps;
            uint4 wv[P];
#pragma unroll
            for (int b = 0; b < P; ++b)
                wv[b] = wnext[b];
            { // weight words of the wave's next item: in this pass, else the first of the next pass
                int jn = j + NW, tbase = t0;
                if (jn >= items) {
                    jn = wid;
                    tbase = t0 + tiles_per_pass;
                }
                const int tpn = min(tiles_per_pass, TW - tbase);
                const int tln = jn / steps, stn = jn - tln * steps;
                load_weight_words<P>(wnext, a.W, wplane, KW, N, tile_of(tbase + tln), r, stn * 16 + 4 * g, KW,
                                     tpn > 0 && jn < tpn * steps);
            }
            if (tl != cur_tl) {
                if (cur_tl >= 0) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        part[(cur_tl * NW + wid) * 256 + (4 * g + e) * 16 + r] = facc[e];
                }
                facc[0] = facc[1] = facc[2] = facc[3] = 0.f;
                cur_tl = tl;
            }
            v4i bops[8];
            int unused_sum;
            expand_weight_words<P, WMODE, false>(wv, bops, unused_sum);
            const int n = min(tile_of(t0 + tl) * 16 + r, N - 1);
            const float *wsc = a.w_scale + (size_t)n * groups;
            const float *wzp = a.w_zero ? a.w_zero + (size_t)n * groups : nullptr;
#pragma unroll
            for (int gsel = 0; gsel < 4; ++gsel) {
                const int blk = 4 * st + gsel; // the 128-element block lane group gsel holds
                if (blk >= blocks)
                    break; // uniform: partial last step
                const unsigned char *xw = (g == gsel) ? xrow + st * 512 : zero_page;
                v4i lo = { 0, 0, 0, 0 }, hi = { 0, 0, 0, 0 };
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(*reinterpret_cast<const v4i *>(xw + i * 16), bops[i], lo, 0, 0, 0);
#pragma unroll
                for (int i = 4; i < 8; ++i)
                    hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(*reinterpret_cast<const v4i *>(xw + i * 16), bops[i], hi, 0, 0, 0);
                if (!g64) {
                    const float sw = wsc[blk];
                    const float zs = wzp ? sw * wzp[blk] : 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        facc[e] += (sw * unshift) * (float)(lo[e] + hi[e]) - zs * sxg[(4 * g + e) * groups + blk];
                } else {
                    const float s0 = wsc[2 * blk], s1 = wsc[2 * blk + 1];
                    const float z0 = wzp ? s0 * wzp[2 * blk] : 0.f, z1 = wzp ? s1 * wzp[2 * blk + 1] : 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float *sx = sxg + (4 * g + e) * groups + 2 * blk;
                        facc[e] += (s0 * unshift) * (float)lo[e] + (s1 * unshift) * (float)hi[e] - z0 * sx[0] - z1 * sx[1];
                    }
                }
            }
        }
        if (cur_tl >= 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                part[(cur_tl * NW + wid) * 256 + (4 * g + e) * 16 + r] = facc[e];
        }
        __syncthreads();
        // output: thread (tile, row i, column c) sums the waves' partial tiles in a fixed order
        for (int u = tid; u < tp * 256; u += NT) {
            const int tl = u >> 8, i = (u >> 4) & 15, c = u & 15;
            const int nn = tile_of(t0 + tl) * 16 + c;
            if (i < Mb && nn < N && !(a.act && (tl & 1))) {
                float v = 0.f;
#pragma unroll
                for (int w2 = 0; w2 < NW; ++w2)
                    v += part[(tl * NW + w2) * 256 + (u & 255)];
                if (a.x_zero)
                    v -= a.x_zero[m0 + i] * a.w_zero_term[nn];
                v *= a.x_scale[m0 + i];
                if (a.act) { // this tile holds gate rows, the next one their up rows
                    float up = 0.f;
#pragma unroll
                    for (int w2 = 0; w2 < NW; ++w2)
                        up += part[((tl + 1) * NW + w2) * 256 + (u & 255)];
                    if (a.x_zero)
                        up -= a.x_zero[m0 + i] * a.w_zero_term[nn + 16];
                    up *= a.x_scale[m0 + i];
                    reinterpret_cast<_Float16 *>(a.D)[(size_t)(m0 + i) * (N / 2) + (nn >> 5) * 16 + c] = (_Float16)(silu(v) * up);
                } else {
                    reinterpret_cast<_Float16 *>(a.D)[(size_t)(m0 + i) * N + nn] = (_Float16)v;
                }
            }
        }
        __syncthreads();
    }
}

template <int Q, int P, bool SIGNED>
static hipError_t launch_decode_grouped(const GemmArgs &a, hipStream_t stream)
{
    if (Int8ModeOf<Q, SIGNED>::value == kFlip || Int8ModeOf<P, SIGNED>::value == kFlip)
        return hipErrorInvalidValue;
    const size_t base = decode_grouped_lds(a.M, a.K, a.group_size); // with one tile per pass
    if (!base || (a.group_size != 64 && a.group_size != 128))
        return hipErrorInvalidValue;
    if (a.act && a.N % 32 != 0)
        return hipErrorInvalidValue;
    const int unit = a.act ? 2 : 1; // tiles that must stay together
    const int units = (a.N + 15) / 16 / unit;
    const int gx = units < 256 ? units : 256;
    const int tpw = unit * ((units + gx - 1) / gx);
    // as many tiles per pass as the rest of the LDS holds (16 KiB of per-wave partial tiles each)
    int tpp = 1 + (int)((160 * 1024 - base) / ((size_t)kDecodeGroupedWaves * 1024));
    if (tpp > tpw)
        tpp = tpw;
    tpp -= tpp % unit;
    if (tpp == 0)
        return hipErrorInvalidValue; // a gate / up pair does not fit beside the activations
    const size_t lds = base + (size_t)(tpp - 1) * kDecodeGroupedWaves * 1024;
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void *>(&gemm_decode_grouped<Q, P, SIGNED>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    const dim3 grid(gx, (a.M + 15) / 16);
    hipLaunchKernelGGL((gemm_decode_grouped<Q, P, SIGNED>), grid, dim3(64 * kDecodeGroupedWaves), lds, stream, a, tpw, tpp);
    return hipGetLastError();
}

static const KernelEntry kSignedGrouped[] = { { 16, 1, 1, 1, 1, kDecodeGroupedWaves, 3, &launch_decode_grouped<ABQ_Q, ABQ_P, true>, 512 } };
static const KernelEntry kUnsignedGrouped[] = { { 16, 1, 1, 1, 1, kDecodeGroupedWaves, 3, &launch_decode_grouped<ABQ_Q, ABQ_P, false>, 512 } };

// Native tile space of this kernel: waves per workgroup.  Entries reuse the MFMA tuple
// (16-row tiles, K split over the waves) with nstage = 3 marking the LDS-staged activations.
// (waves, plane words per lane and item)
#define ABQ_DECODE_VARIANTS(V) V(4, 4) V(8, 4) V(16, 4) V(16, 2)

#define ABQ_ENTRY_T(NW, SW) { 16, 1, 1, 1, 1, NW, 3, &launch_mfma_decode<ABQ_Q, ABQ_P, true, NW, SW>, 128 * SW },
#define ABQ_ENTRY_F(NW, SW) { 16, 1, 1, 1, 1, NW, 3, &launch_mfma_decode<ABQ_Q, ABQ_P, false, NW, SW>, 128 * SW },

static const KernelEntry kSigned[] = { ABQ_DECODE_VARIANTS(ABQ_ENTRY_T) };
static const KernelEntry kUnsigned[] = { ABQ_DECODE_VARIANTS(ABQ_ENTRY_F) };

#define ABQ_CAT_(a, b, c, d) a##b##c##d
#define ABQ_CAT(a, b, c, d) ABQ_CAT_(a, b, c, d)

void ABQ_CAT(abq_decode_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSigned, (int)(sizeof(kSigned) / sizeof(kSigned[0])) };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsigned, (int)(sizeof(kUnsigned) / sizeof(kUnsigned[0])) };
}

void ABQ_CAT(abq_decode_grouped_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSignedGrouped, 1 };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsignedGrouped, 1 };
}

} // namespace abq
