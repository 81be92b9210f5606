// Internal interface between the host API (abq_api.cpp) and the HIP kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "abq_bits.h"

namespace abq {

// Arguments of every GEMM kernel (the reference passes AqBMMAOpState::Argument_t,
// engine/mma_any/aq_bmma_op.h:24-31).
struct GemmArgs {
    const uint32_t *X; // planes [x_bits][M][KW]
    const uint32_t *W; // planes [w_bits][N][KW]
    void *D;           // [M][N] int32 or fp16
    const void *C;     // one fp16 scale (ABQ_OUT_F16_TENSOR) or null
    const float *x_scale;
    const float *w_scale;
    int M, N, K, KW; // KW = K / 32 plane words per row
    int out_kind;
    int group_size;
    int lpr_log2;    // popcount kernels: log2(lanes that share one weight row)
    int act;                 // 0: none; 1: SiLU gate (group-scale kernels): rows of W are gate / up blocks of 16,
                             // D[m][16 b + c] = silu(out[m][32 b + c]) * out[m][32 b + 16 + c], D is [M][N / 2]
    // zero points of the group-scale path (all optional)
    const float *w_zero;       // [N][K/group_size], in units of weight codes
    const float *x_zero;       // [M], in units of activation codes
    const int *x_group_sums;   // [M][K/group_size] sums of activation codes (needed with w_zero)
    const float *w_zero_term;  // [N] sum_g w_scale * (sum of weight codes - group_size * w_zero) (needed with x_zero)
    const float *x_pack_scale; // kernels that quantise fp16 activations themselves: X is fp16 [M][K], this the static scale
    int x_dynamic;             // ... or, per token from the rows' own extrema: 1 symmetric, 2 with a zero point; 0: not
    // sums over K of the unsigned codes of every row, for kernels that feed an unsigned 8-bit operand as value - 128
    // and take no sums themselves (entries with kNeedsRowSums): D = acc + 128 (w sums if X is 8 bits wide)
    // + 128 (x sums if W is) - 2^14 K (if both are)
    const int *x_row_sums;     // [M]
    const int *w_row_sums;     // [N]
    // the decode kernel on prepared operands, unsigned pairs: whether the 8-bit records of X (W) hold codes up to 255
    // (fed as value - 128, with the row sums above) or padded narrower codes, which are fed as they are
    int flip_x, flip_w;
};

typedef hipError_t (*GemmLauncher)(const GemmArgs &, hipStream_t);

// One kernel instantiation together with the tile tuple that names it.
struct KernelEntry {
    int mi;                 // MFMA rows (16 / 32); 1 for the popcount kernels
    int tm, tn;             // MFMA tiles per wave (popcount: tm = activation rows per pass)
    int wm, wn, wk;         // waves per workgroup along M, N, K
    int nstage;
    GemmLauncher launch;
    int kb;                 // K elements per LDS stage (tiled kernel); 0 where it does not apply
    size_t lds;             // dynamic LDS of the launch where the kernel fixes it itself; 0: derived from the tile
    int flags;              // kNeedsRowSums: reads GemmArgs::x_row_sums / w_row_sums; the entry of the same tile tuple
                            // in front of it in the table is the kernel that runs when the sums are not to be had
};
constexpr int kNeedsRowSums = 1;

struct KernelTable {
    int x_bits, w_bits, is_signed;
    const KernelEntry *entries;
    int count;
};

// Defined once per (x_bits, w_bits) translation unit; looked up by abq_api.cpp.
const KernelTable *mfma_tables(int *count);
const KernelTable *bcnt_tables(int *count);
hipError_t launch_bcnt_generic(const GemmArgs &, int x_bits, int w_bits, int is_signed, hipStream_t);

// Waves per workgroup of the decode kernel with group scales, and the LDS it needs (per-wave partial
// tiles, the activation group sums, a page of zeros, the expanded activations); 0 if that exceeds a
// compute unit's LDS.
constexpr int kDecodeGroupedWaves = 16;
inline size_t decode_grouped_lds(int M, int K, int group_size)
{
    const int mb = M < 16 ? M : 16;
    const int row = (K + 511) / 512 * 512 + 16; // an expanded row, padded to whole 512-element steps
    const size_t need = (size_t)kDecodeGroupedWaves * 256 * 4 + (size_t)16 * (K / group_size) * 4 + 128 + (size_t)mb * row;
    return need <= 160 * 1024 ? need : 0;
}

// Decode kernel on K-tiled operands (abq_gemm_decode_tiled.hip): LDS of one workgroup = per-wave partial tiles,
// then the activations of its rows (one K tile of slack for the ragged last step, whole wave loads), and the
// rows per workgroup (up to 16) that keep it within a compute unit's LDS; 0 if not even one row fits.
inline size_t decode_tiled_lds(int nw, int t, int mrows, int K, int q)
{
    return (size_t)nw * t * 1024 + (size_t)mrows * (K / 128 + 1) * q * 16 + 1024;
}
inline int decode_tiled_rows(int nw, int t, int M, int K, int q)
{
    int mrows = M < 16 ? M : 16;
    while (mrows > 1 && decode_tiled_lds(nw, t, mrows, K, q) > 150 * 1024)
        mrows = (mrows + 1) / 2;
    return decode_tiled_lds(nw, t, mrows, K, q) <= 160 * 1024 ? mrows : 0;
}

// The same kernel with group scales (groups of 128 = one K tile): fp32 partial tiles, and after the activations the
// tile's weight scales and zero points ([group][16 rows] each, T tiles) and the activation group sums
// ([group][16 rows]), every array padded to whole wave loads of four bytes per lane.
// (group: 128, or 64 = two scale groups per K tile)
inline size_t decode_tiled_grouped_lds(int nw, int t, int mrows, int K, int q, int group = 128)
{
    const size_t groups = (size_t)K / group;
    const size_t per_tile = (groups * 16 + 63) / 64 * 256; // bytes of one [group][16] float array
    return decode_tiled_lds(nw, t, mrows, K, q) + (2 * t + 1) * per_tile + 1024;
}
inline int decode_tiled_grouped_rows(int nw, int t, int M, int K, int q, int group = 128)
{
    int mrows = M < 16 ? M : 16;
    while (mrows > 1 && decode_tiled_grouped_lds(nw, t, mrows, K, q, group) > 150 * 1024)
        mrows = (mrows + 1) / 2;
    return decode_tiled_grouped_lds(nw, t, mrows, K, q, group) <= 160 * 1024 ? mrows : 0;
}

// Workgroup id -> output tile.  XCD x = id % 8 owns n blocks [x * npx, (x + 1) * npx); inside an XCD the
// workgroups run through groups of four m blocks, M fastest inside a group, then N, then the next group:
// the 32 or 64 workgroups an XCD runs at a time then cover a patch of 4 x 8 (or 4 x 16) tiles, so every
// activation and weight block they load is shared in that XCD's L2, whatever M is (with M fastest over
// all m blocks, 16384 rows ran 25-35 % slower; groups of 2, 4 and 8 measured within 2 %, 4 ahead by up
// to 4 % at 2048 rows).
__device__ __forceinline__ void tile_of_workgroup(int id, int m_blocks, int n_blocks_per_xcd, int *mb, int *nb)
{
    constexpr int GM = 4;
    const int xcd = id & 7, slot = id >> 3;
    const int per_group = GM * n_blocks_per_xcd;
    const int grp = slot / per_group, in = slot - grp * per_group;
    const int gm = min(GM, m_blocks - grp * GM); // the last group may be short
    *mb = grp * GM + in % gm;
    *nb = xcd * n_blocks_per_xcd + in / gm;
}

// ---- byte shuffles inside a quad of lanes (the packing kernels and the decode kernel that quantises its own
// activations assemble K-tiled 8-bit records with them) ------------------------------------------------

// The low bytes of four integers as one dword, a in byte 0.
__device__ __forceinline__ uint32_t pack_low_bytes(int a, int b, int c, int d)
{
    const uint32_t ab = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
    const uint32_t cd = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// 4 x 4 byte transpose across a quad with the lane order reversed: lane s returns the dword whose byte c is
// byte s of lane 3 - c's argument.  sel_pair / sel_half are the lane's byte selectors of the two exchange
// steps (quad_transpose_selectors).
__device__ __forceinline__ uint32_t quad_transpose_bytes(uint32_t v, uint32_t sel_pair, uint32_t sel_half)
{
    const uint32_t p = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true); // lane ^ 1
    const uint32_t x = __builtin_amdgcn_perm(p, v, sel_pair);
    const uint32_t q = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, true); // lane ^ 2
    return __builtin_amdgcn_perm(q, x, sel_half);
}

__device__ __forceinline__ void quad_transpose_selectors(int quad_lane, uint32_t &sel_pair, uint32_t &sel_half)
{
    // step 1: even lanes keep their bytes 0, 2 and take the partner's 0, 2; odd lanes the bytes 1, 3
    sel_pair = (quad_lane & 1) ? 0x03070105u : 0x06020400u;
    // step 2: lanes 0, 1 take the low halves, lanes 2, 3 the high halves, bytes in reversed order
    sel_half = (quad_lane & 2) ? 0x06070203u : 0x00010405u;
}

// x * sigmoid(x), the reciprocal by the hardware instruction (1 ulp) instead of the division sequence
__device__ __forceinline__ float silu(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// ---- output stage shared by all kernels ------------------------------------------------
// out_kind values mirror abq_out_kind in include/abq_gemm.h.
__device__ __forceinline__ void store_result(const GemmArgs &a, int m, int n, int acc)
{
    const size_t idx = (size_t)m * a.N + n;
    if (a.out_kind == 0) {
        reinterpret_cast<int *>(a.D)[idx] = acc;
    } else if (a.out_kind == 1) {
        // half(acc) * scale, both steps rounding to fp16
        // (fastertransformer/.../abqgemm/mma_any/aq_bmma_kernel.h:516-519 of the reference).
        // int -> float -> half rounds once: beyond 2^24, where the first step is inexact,
        // the half result is infinity either way.
        const _Float16 scale = *reinterpret_cast<const _Float16 *>(a.C);
        const _Float16 h = (_Float16)(float)acc;
        reinterpret_cast<_Float16 *>(a.D)[idx] = h * scale;
    } else if (a.out_kind == 3) {
        // the same with the scale held as one float: converted to fp16 first, then as above
        const _Float16 scale = (_Float16)*reinterpret_cast<const float *>(a.C);
        const _Float16 h = (_Float16)(float)acc;
        reinterpret_cast<_Float16 *>(a.D)[idx] = h * scale;
    } else {
        const float r = (float)acc * a.x_scale[m] * a.w_scale[n];
        reinterpret_cast<_Float16 *>(a.D)[idx] = (_Float16)r;
    }
}

// Out-of-line fp16 store for kernels whose epilogue stores hundreds of elements per lane: keeps
// the unrolled epilogue small (the int32 store is inlined, the fp16 variants are a call).  The
// operands travel by value so that the kernel's argument block never has its address taken
// (which would push every later read of it through memory).
struct StoreOperands {
    void *D;
    const void *C;
    const float *x_scale;
    const float *w_scale;
    int N;
    int out_kind;
};

__device__ __forceinline__ StoreOperands store_operands(const GemmArgs &a)
{
    return StoreOperands{ a.D, a.C, a.x_scale, a.w_scale, a.N, a.out_kind };
}

__device__ __attribute__((noinline)) static void store_result_call(void *D, const void *C, const float *x_scale,
                                                                   const float *w_scale, int N, int out_kind, int m,
                                                                   int n, int acc)
{
    GemmArgs a;
    a.D = D;
    a.C = C;
    a.x_scale = x_scale;
    a.w_scale = w_scale;
    a.N = N;
    a.out_kind = out_kind;
    store_result(a, m, n, acc);
}

__device__ __forceinline__ void store_result_compact(const StoreOperands &o, int m, int n, int acc)
{
    if (o.out_kind == 0)
        __builtin_nontemporal_store(acc, reinterpret_cast<int *>(o.D) + ((size_t)m * o.N + n));
    else
        store_result_call(o.D, o.C, o.x_scale, o.w_scale, o.N, o.out_kind, m, n, acc);
}

} // namespace abq
