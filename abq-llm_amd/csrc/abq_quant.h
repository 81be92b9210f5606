// Per-token dynamic quantisation of fp16 activations: what a row's codes follow from once its extrema are known.
// Shared by the quantise-and-pack kernels (abq_pack.hip) and the decode kernel that quantises its activations
// itself (abq_gemm_decode_tiled.hip), so that both produce the same codes bit for bit.
// Semantics: algorithm/quantize/quantizer.py:111-179 of the reference (per_token_dynamic_calibration, fake_quant).
#pragma once
#include <hip/hip_runtime.h>

namespace abq {

// What a row's quantisation needs once its minimum and maximum are known.
struct QuantRow {
    float scale, recip, zp_stored, lo_stored, hi_stored, zero_out;
};

// scale, zero point and code range of a row from its extrema (formulas in the comment above)
__device__ __forceinline__ QuantRow quant_row_params(float mx, float mn, int bits, int symmetric)
{
    const int half_range = 1 << (bits - 1);
    float scale, zp;
    int lo, hi;
    if (symmetric) {
        scale = fmaxf(fabsf(mx), fabsf(mn)) / (float)(half_range - 1);
        scale = fminf(fmaxf(scale, 1e-5f), 1e4f);
        zp = 0.f;
        lo = -half_range;
        hi = half_range - 1;
    } else {
        scale = (mx - mn) / (float)(2 * half_range - 1);
        scale = fminf(fmaxf(scale, 1e-5f), 1e4f);
        zp = rintf(fminf(fmaxf(-mn / scale, -1e4f), 1e4f));
        lo = 0;
        hi = 2 * half_range - 1;
    }
    QuantRow q;
    q.scale = scale;
    // x / scale in three operations instead of the dozen of a full division, with the same bits: recip is the
    // correctly rounded reciprocal (the fp64 quotient is never close enough to an fp32 midpoint for the second
    // rounding to cross it), t = x recip is within an ulp of the quotient, the residual x - t scale is exact in
    // an fma, and t + residual recip then rounds to the quotient itself (checked against the division on a CPU
    // for every finite fp16 value and 600 000 scales of the forms above; a zero may come out with the other
    // sign, which the rounding to an integer code forgets).  div_fixup restores what a division makes of an
    // infinite x.
    q.recip = (float)(1.0 / (double)scale);
    // rint(q) + zp, clamped to [lo, hi], minus the offset of the stored code: the offset is taken off before the
    // clamp instead (all three are small integers, so the sums are the same numbers)
    const float code_offset = symmetric ? 0.f : (float)half_range;
    q.zp_stored = zp - code_offset;
    q.lo_stored = (float)lo - code_offset;
    q.hi_stored = (float)hi - code_offset;
    q.zero_out = symmetric ? 0.f : zp - (float)half_range;
    return q;
}

// The stored code of one element: rint(x / scale) + zero point, clamped to the code range (offsets as in
// quant_row_params).  The fix-up only matters for an infinite x, but one more instruction per element is cheaper
// than a branch around it.
__device__ __forceinline__ int quant_code(float xf, const QuantRow &q)
{
    const float t = xf * q.recip;
    const float quotient = __builtin_amdgcn_div_fixupf(__builtin_fmaf(__builtin_fmaf(-t, q.scale, xf), q.recip, t), q.scale, xf);
    return (int)__builtin_amdgcn_fmed3f(rintf(quotient) + q.zp_stored, q.lo_stored, q.hi_stored);
}

} // namespace abq
