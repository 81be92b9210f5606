/*
 * CPU oracle for the arbitrary-bit quantized GEMM path.  TEST INFRASTRUCTURE ONLY:
 * it is linked or loaded by tests/, by the smoke check and by the CPU-baseline leg of
 * the benchmark, never by the shipped library.
 *
 * Every function restates one piece of the reference engine and cites the lines it
 * follows (paths are relative to the reference tree).
 *
 * Layout vocabulary (same as the reference):
 *   planes   uint32 words, K-major.  planes[b][r][j] holds bit b of the 32 elements
 *            in[r][32*j .. 32*j+31]; element e of the group sits at bit (31 - e).
 *   X planes [x_bits][M][K/32], W planes [w_bits][N][K/32], D row-major [M][N].
 *
 * Pinning status of each function is listed in the header comment of abq_oracle.c.
 */
#ifndef ABQ_ORACLE_H
#define ABQ_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* engine/common/pack.cu:46-64 (kernel pack) + :93-104 (launch_pack) */
void abq_oracle_pack_i32(const int32_t *in, uint32_t *planes, int rows, int k, int bits);

/* engine/common/pack.cu:18-44 (kernel pack4) + :73-84 (launch_pack4).
 * in: rows*k/8 words, eight 4-bit elements per word, first element in the top nibble. */
void abq_oracle_pack_u4(const uint32_t *in, uint32_t *planes, int rows, int k, int bits);

/* fastertransformer/src/fastertransformer/kernels/abqgemm/abq_gemm_wrapper.cu:29-54 (pack_half):
 * v = (int)( half(x) * half(scale) ), product rounded to fp16 first, conversion truncates. */
void abq_oracle_pack_f16(const uint16_t *in_half_bits, float scale, uint32_t *planes, int rows,
                         int k, int bits);

/* inverse of the plane layout; is_signed sign-extends from bit (bits-1). */
void abq_oracle_unpack(const uint32_t *planes, int32_t *out, int rows, int k, int bits,
                       int is_signed);

/* engine/test_any_mma.cu:58-84 (compute_ref), loop for loop: single thread, bit serial. */
void abq_oracle_gemm_bitserial(const uint32_t *w_planes, const uint32_t *x_planes, int32_t *d,
                               int M, int N, int K, int w_bits, int x_bits, int is_signed);

/* same sum as compute_ref, one popcount(x & w) per word pair, OpenMP over (m, n).
 * threads <= 0 means "all host cores". Returns the thread count used. */
int abq_oracle_gemm_popc(const uint32_t *w_planes, const uint32_t *x_planes, int32_t *d, int M,
                         int N, int K, int w_bits, int x_bits, int is_signed, int threads);

/* closed form D = Xint * Wint^T on unpacked integers, int64 accumulate.
 * Returns 0, or 1 if some result does not fit int32. */
int abq_oracle_gemm_int(const int32_t *x, const int32_t *w, int32_t *d, int M, int N, int K);

/* FT epilogue, abqgemm/mma_any/aq_bmma_kernel.h:479,516-519:
 * D = __int2half_rn(acc) * scale, both steps round to fp16 (nearest even). */
void abq_oracle_epilogue_f16(const int32_t *acc, uint16_t scale_half_bits, uint16_t *d_half_bits,
                             int count);

/* fp16 helpers (software, IEEE binary16, round to nearest even) */
uint16_t abq_oracle_f32_to_f16(float f);
float abq_oracle_f16_to_f32(uint16_t h);

#ifdef __cplusplus
}
#endif
#endif
