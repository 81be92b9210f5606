/*
 * CPU oracle for the arbitrary-bit quantized GEMM path -- TEST INFRASTRUCTURE ONLY.
 * Nothing in the shipped library may include, link or load this file; it exists so that
 * tests, the smoke check and the benchmark's CPU-baseline leg have something independent
 * to compare the HIP kernels with.
 *
 * What each function follows in the reference, and what pins it (the checks live in
 * tests/test_oracle.py):
 *
 *   abq_oracle_pack_i32        engine/common/pack.cu:46-64,93-104
 *       pinned by hand-written vectors, the closed form "bit (31-e) of word j of plane b
 *       is bit b of in[32j+e]" evaluated independently in numpy, and pack->unpack round trip.
 *   abq_oracle_pack_u4         engine/common/pack.cu:18-44,73-84
 *       pinned by equivalence with pack_i32 on nibble-packed copies of the same values
 *       and a hand vector.
 *   abq_oracle_pack_f16        fastertransformer/.../abqgemm/abq_gemm_wrapper.cu:29-54
 *       pinned by a sweep over all 65536 fp16 bit patterns against numpy float16
 *       arithmetic (np.float16 multiply, truncation) for several scales.
 *   abq_oracle_gemm_bitserial  engine/test_any_mma.cu:58-84
 *   abq_oracle_gemm_popc       same sum, word popcounts
 *   abq_oracle_gemm_int        textbook integer GEMM
 *       the three are pinned against each other, against numpy int64 matmul of the
 *       unpacked integers, against all-ones / single-bit special cases and against brute
 *       force over all value pairs for small bit widths.
 *   abq_oracle_epilogue_f16    fastertransformer/.../abqgemm/mma_any/aq_bmma_kernel.h:479,516-519
 *       pinned against numpy float16 arithmetic.
 *
 * No function here is "parity unpinned".
 */
#include "abq_oracle.h"

#include <math.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 helpers */

static uint16_t double_to_f16(double d)
{
    uint16_t sign = (uint16_t)(signbit(d) ? 0x8000u : 0u);
    if (isnan(d))
        return (uint16_t)(sign | 0x7e00u);
    double a = fabs(d);
    if (a >= 65520.0) /* halfway between 65504 and 2^16 rounds to even = overflow */
        return (uint16_t)(sign | 0x7c00u);
    if (a < 6.103515625e-05) { /* below 2^-14: subnormal, unit 2^-24 */
        double m = rint(a * 16777216.0);
        return (uint16_t)(sign | (uint16_t)m);
    }
    int ex;
    (void)frexp(a, &ex); /* a = f * 2^ex, f in [0.5, 1) */
    int e = ex - 1;
    double m = rint(ldexp(a, 10 - e)); /* in [1024, 2048] */
    if (m >= 2048.0) {
        m = 1024.0;
        e += 1;
    }
    if (e + 15 >= 31)
        return (uint16_t)(sign | 0x7c00u);
    return (uint16_t)(sign | (uint16_t)((e + 15) << 10) | (uint16_t)((int)m - 1024));
}

uint16_t abq_oracle_f32_to_f16(float f)
{
    return double_to_f16((double)f);
}

float abq_oracle_f16_to_f32(uint16_t h)
{
    int sign = (h >> 15) & 1;
    int e = (h >> 10) & 0x1f;
    int m = h & 0x3ff;
    double v;
    if (e == 0)
        v = ldexp((double)m, -24);
    else if (e == 31)
        v = m ? NAN : INFINITY;
    else
        v = ldexp((double)(m + 1024), e - 25);
    return (float)(sign ? -v : v);
}

/* half * half as the device computes it: exact product (fits a float), one rounding. */
static uint16_t f16_mul(uint16_t a, uint16_t b)
{
    double p = (double)abq_oracle_f16_to_f32(a) * (double)abq_oracle_f16_to_f32(b);
    return double_to_f16(p);
}

/* half -> int, round toward zero; NaN gives 0, out-of-range saturates (device rule). */
static int32_t f16_to_int_rz(uint16_t h)
{
    float f = abq_oracle_f16_to_f32(h);
    if (isnan(f))
        return 0;
    if (isinf(f))
        return f > 0 ? INT32_MAX : INT32_MIN;
    return (int32_t)truncf(f);
}

/* ------------------------------------------------------------------ packing */

void abq_oracle_pack_i32(const int32_t *in, uint32_t *planes, int rows, int k, int bits)
{
    /* pack.cu:48-63: one output word per (bit, idx); the word gathers 32 consecutive
     * int32 inputs, input e lands on bit 31-e.  The reference reads them as 8 uint4
     * (i = 0..7, lanes x,y,z,w -> e = 4i, 4i+1, 4i+2, 4i+3). */
    const long L = (long)rows * (k / 32);
    for (int bit = 0; bit < bits; ++bit) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static) if (L > 65536)
#endif
        for (long idx = 0; idx < L; ++idx) {
            uint32_t word = 0;
            for (int i = 0; i < 8; ++i) {
                const uint32_t *v = (const uint32_t *)in + idx * 32 + i * 4;
                word |= ((v[0] >> bit) & 1u) << (32 - 1 - i * 4);
                word |= ((v[1] >> bit) & 1u) << (32 - 2 - i * 4);
                word |= ((v[2] >> bit) & 1u) << (32 - 3 - i * 4);
                word |= ((v[3] >> bit) & 1u) << (32 - 4 - i * 4);
            }
            planes[bit * L + idx] = word;
        }
    }
}

void abq_oracle_pack_u4(const uint32_t *in, uint32_t *planes, int rows, int k, int bits)
{
    /* pack.cu:20-43: one uint4 (4 words, 32 nibbles) per output word; within a word the
     * first element is the highest nibble: element b of word c uses shift (7 - b%8)*4. */
    const long L = (long)rows * k / 32;
    for (int bit = 0; bit < bits; ++bit) {
        for (long idx = 0; idx < L; ++idx) {
            uint32_t word = 0;
            for (int b = 0; b < 32; ++b) {
                uint32_t src = in[idx * 4 + b / 8];
                uint32_t nib = src >> ((8 - 1 - (b % 8)) * 4);
                word |= ((nib >> bit) & 1u) << (32 - 1 - b);
            }
            planes[bit * L + idx] = word;
        }
    }
}

void abq_oracle_pack_f16(const uint16_t *in_half_bits, float scale, uint32_t *planes, int rows,
                         int k, int bits)
{
    /* abq_gemm_wrapper.cu:33-53: scale is converted to half once per use, the product is
     * a half multiply, static_cast<int> truncates; no clamp to the bit width, so values
     * outside it alias.  Element 8i+c of a 32-group lands on bit 31-(8i+c). */
    const long L = (long)rows * (k / 32);
    const uint16_t hs = abq_oracle_f32_to_f16(scale);
    for (int bit = 0; bit < bits; ++bit) {
        for (long idx = 0; idx < L; ++idx) {
            uint32_t word = 0;
            for (int e = 0; e < 32; ++e) {
                int32_t v = f16_to_int_rz(f16_mul(in_half_bits[idx * 32 + e], hs));
                word |= (((uint32_t)v >> bit) & 1u) << (31 - e);
            }
            planes[bit * L + idx] = word;
        }
    }
}

void abq_oracle_unpack(const uint32_t *planes, int32_t *out, int rows, int k, int bits,
                       int is_signed)
{
    const long L = (long)rows * (k / 32);
#ifdef _OPENMP
#pragma omp parallel for schedule(static) if (L > 65536)
#endif
    for (long idx = 0; idx < L; ++idx) {
        for (int e = 0; e < 32; ++e) {
            uint32_t v = 0;
            for (int bit = 0; bit < bits; ++bit)
                v |= ((planes[bit * L + idx] >> (31 - e)) & 1u) << bit;
            int32_t s = (int32_t)v;
            if (is_signed && bits < 32 && (v >> (bits - 1)) & 1u)
                s -= (int32_t)(1u << bits);
            out[idx * 32 + e] = s;
        }
    }
}

/* ------------------------------------------------------------------ GEMM */

static int int_pow2(int exp) /* test_any_mma.cu:39-49 with base 2 */
{
    int result = 1, base = 2;
    while (exp) {
        if (exp % 2)
            result *= base;
        exp /= 2;
        base *= base;
    }
    return result;
}

void abq_oracle_gemm_bitserial(const uint32_t *w, const uint32_t *x, int32_t *d, int M, int N,
                               int K, int w_bits, int x_bits, int is_signed)
{
    /* test_any_mma.cu:60-83.  The reference extracts bit k with signed shifts (bit 31
     * comes out as -1 for both operands, whose product is again +1); unsigned shifts
     * give the same products without relying on that. */
    const long KW = K / 32;
    for (int m = 0; m < M; m++) {
        for (int n = 0; n < N; n++) {
            int tmp = 0;
            for (int xb = 0; xb < x_bits; xb++) {
                int xm = is_signed && (xb == x_bits - 1) ? -1 * int_pow2(xb) : int_pow2(xb);
                for (int wb = 0; wb < w_bits; wb++) {
                    int wm = is_signed && (wb == w_bits - 1) ? -1 * int_pow2(wb) : int_pow2(wb);
                    for (long kt = 0; kt < KW; kt++) {
                        uint32_t w_int = w[(long)wb * N * KW + n * KW + kt];
                        uint32_t x_int = x[(long)xb * M * KW + m * KW + kt];
                        for (int k = 0; k < 32; k++) {
                            int x_val = (int)((x_int >> k) & 1u);
                            int w_val = (int)((w_int >> k) & 1u);
                            tmp += xm * wm * x_val * w_val;
                        }
                    }
                }
            }
            d[(long)m * N + n] = tmp;
        }
    }
}

int abq_oracle_gemm_popc(const uint32_t *w, const uint32_t *x, int32_t *d, int M, int N, int K,
                         int w_bits, int x_bits, int is_signed, int threads)
{
    const long KW = K / 32;
    int used = 1;
#ifdef _OPENMP
    used = threads > 0 ? threads : omp_get_max_threads();
#pragma omp parallel for collapse(2) schedule(static) num_threads(used)
#endif
    for (int m = 0; m < M; m++) {
        for (int n = 0; n < N; n++) {
            int64_t acc = 0;
            for (int xb = 0; xb < x_bits; xb++) {
                const uint32_t *xr = x + (long)xb * M * KW + (long)m * KW;
                for (int wb = 0; wb < w_bits; wb++) {
                    const uint32_t *wr = w + (long)wb * N * KW + (long)n * KW;
                    long cnt = 0;
                    for (long kt = 0; kt < KW; kt++)
                        cnt += __builtin_popcount(xr[kt] & wr[kt]);
                    int neg = is_signed && ((xb == x_bits - 1) != (wb == w_bits - 1));
                    int64_t term = (int64_t)cnt << (xb + wb);
                    acc += neg ? -term : term;
                }
            }
            d[(long)m * N + n] = (int32_t)acc;
        }
    }
    (void)threads;
    return used;
}

int abq_oracle_gemm_int(const int32_t *x, const int32_t *w, int32_t *d, int M, int N, int K)
{
    int overflow = 0;
#ifdef _OPENMP
#pragma omp parallel for collapse(2) schedule(static) reduction(| : overflow)
#endif
    for (int m = 0; m < M; m++) {
        for (int n = 0; n < N; n++) {
            int64_t acc = 0;
            const int32_t *xr = x + (long)m * K;
            const int32_t *wr = w + (long)n * K;
            for (int k = 0; k < K; k++)
                acc += (int64_t)xr[k] * wr[k];
            if (acc > INT32_MAX || acc < INT32_MIN)
                overflow |= 1;
            d[(long)m * N + n] = (int32_t)acc;
        }
    }
    return overflow;
}

/* ------------------------------------------------------------------ epilogue */

void abq_oracle_epilogue_f16(const int32_t *acc, uint16_t scale_half_bits, uint16_t *d, int count)
{
    for (int i = 0; i < count; ++i) {
        uint16_t h = double_to_f16((double)acc[i]); /* __int2half_rn */
        d[i] = f16_mul(h, scale_half_bits);
    }
}
