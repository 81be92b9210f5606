/*
 * abq_gemm.h -- C ABI of the MI355X (gfx950) arbitrary-bit quantized GEMM engine.
 *
 * Every entry point takes plain pointers and sizes.  Device pointers must be valid on the
 * current HIP device; `stream` is a hipStream_t passed as void* (NULL = the null stream).
 * The library allocates no device memory in any entry point declared here and keeps no mutable
 * global state besides the table of measured best tiles (abq_tuning_*, guarded by a mutex), so calls
 * are stream ordered and thread safe on distinct states.
 *
 * Data layout (identical to the reference engine, see engine/common/pack.cu:46-64 there):
 *   planes   uint32 words, K-major, MSB first: bit (31-e) of planes[b][r][j] is bit b of
 *            element in[r][32*j+e].   X planes [x_bits][M][K/32], W planes [w_bits][N][K/32].
 *   D        row-major [M][N], int32 or fp16 depending on the output kind.
 *   The GEMM computes D = Xint . Wint^T, i.e.
 *   D[m][n] = sum_{i<x_bits, j<w_bits} s_i s_j 2^(i+j) popcount(Xp[i][m][:] & Wp[j][n][:])
 *   with s = -1 only for the MSB plane of a signed operand.
 *   K must be a multiple of 128 and at least 128 (engine/test_any_mma.cu:99).
 *
 * Each declaration cites the reference interface it replaces (paths relative to the
 * reference tree).
 */
#ifndef ABQ_GEMM_H
#define ABQ_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ABQ_VERSION 1

/* Status codes.  The reference reports errors as cudaError_t from the pack launchers
 * (engine/common/pack.cu:82,102), an initSuccess flag (engine/mma_any/aq_bmma_op.h:23,102,114)
 * and printf + early return in the FT wrapper (abq_gemm_wrapper.cu:100-103,128-136). */
typedef enum abq_status {
    ABQ_OK = 0,
    ABQ_ERR_INVALID_ARG = 1, /* null pointer, non-positive size, bits out of range        */
    ABQ_ERR_BAD_K = 2,       /* K < 128 or K % 128 != 0                                    */
    ABQ_ERR_UNSUPPORTED = 3, /* bit combination / tile tuple / option not implemented      */
    ABQ_ERR_NOT_INITIALIZED = 4, /* exec called on a state whose init failed               */
    ABQ_ERR_LAUNCH = 5,      /* the HIP runtime rejected the launch (see abq_last_hip_error) */
    ABQ_ERR_NO_DEVICE = 6,   /* no usable gfx950 device                                    */
    ABQ_ERR_TOO_LARGE = 7    /* a size exceeds a documented limit                          */
} abq_status;

const char *abq_status_string(abq_status s);
/* hipError_t of the last failed launch on this thread, 0 if none. */
int abq_last_hip_error(void);
int abq_version(void);

/* ---------------------------------------------------------------------------------------
 * Bit-plane packing
 * ------------------------------------------------------------------------------------- */

/* Replaces launch_pack (engine/common/pack.h:23-24, pack.cu:46-64,93-104) and
 * ABQGEMMWrapper::pack(const int*, ...) (abq_gemm_wrapper.cu:9-27,71-77).
 * in: int32 [rows][k] on the device; planes: uint32 [bits][rows][k/32]. k % 32 == 0. */
abq_status abq_pack_i32(const int32_t *in, uint32_t *planes, int rows, int k, int bits,
                        void *stream);

/* Replaces launch_pack4 (engine/common/pack.h:20-21, pack.cu:18-44,73-84).
 * in: uint32 [rows*k/8], eight 4-bit elements per word, first element in the top nibble. */
abq_status abq_pack_u4(const uint32_t *in, uint32_t *planes, int rows, int k, int bits,
                       void *stream);

/* Replaces pack_half / ABQGEMMWrapper::pack(const half*, const float*, ...)
 * (fastertransformer/src/fastertransformer/kernels/abqgemm/abq_gemm_wrapper.cu:29-69).
 * in: fp16 [rows][k]; scale: one float on the device; value = (int)(half(x) * half(scale)),
 * the product rounded to fp16, the conversion truncating, no clamp. */
abq_status abq_pack_f16(const void *in_f16, const float *scale_dev, uint32_t *planes, int rows,
                        int k, int bits, void *stream);

/* ---------------------------------------------------------------------------------------
 * Tile configuration = the tuple encoded in the reference's kernel symbol names
 * (engine/common/base.h:144-146): X_BITS x W_BITS x SIGNED _ BM x BN x BK _ WM x WN x WK _
 * MMA_M x MMA_N x MMA_K _ NSTAGE.
 *
 * The MMA triple selects the gfx950 strategy:
 *   1 x 1 x 128   VALU AND + popcount, K along the lanes, wavefront reduction
 *   16 x 16 x 64  planes re-assembled to int8 in registers, v_mfma_i32_16x16x64_i8
 *                 (NSTAGE = 3: decode kernel, activations staged in LDS; NSTAGE = 2: every wave
 *                 expands its own activations; NSTAGE = 6: decode kernel on K-tiled operands,
 *                 BN / 16 weight tiles per workgroup, WK = K elements a wave keeps in flight)
 *   32 x 32 x 32  the same feeding v_mfma_i32_32x32x32_i8 (NSTAGE = 4: LDS-staged kernels on K-tiled
 *                 operands, WK = 128 (or 64) = K elements per LDS stage and group of waves; BK = 2 WK:
 *                 two groups of waves share the tile and split K between them, for small grids)
 * Any other triple (the reference's 8x8x128, 16x8x128, 16x8x256 tensor-core shapes) asks the
 * library to choose strategy and tile itself from (bits, M, N, K).
 * ------------------------------------------------------------------------------------- */
typedef struct abq_tile_config {
    int x_bits, w_bits, is_signed;
    int block_m, block_n, block_k;
    int warp_m, warp_n, warp_k;
    int mma_m, mma_n, mma_k;
    int nstage;
} abq_tile_config;

typedef enum abq_strategy {
    ABQ_STRATEGY_AUTO = 0,
    ABQ_STRATEGY_BCNT = 1,   /* VALU popcount          */
    ABQ_STRATEGY_MFMA16 = 2, /* int8 MFMA 16x16x64     */
    ABQ_STRATEGY_MFMA32 = 3, /* int8 MFMA 32x32x32     */
    ABQ_STRATEGY_GENERIC = 4, /* any 1..16 bit pair, runtime loops (slow, always available) */
    ABQ_STRATEGY_DECODE = 5,  /* int8 MFMA 16x16x64, activations expanded once per workgroup
                                 into LDS, persistent grid; tile tuples with NSTAGE = 3       */
    ABQ_STRATEGY_TILED = 6,   /* int8 MFMA 32x32x32, LDS-staged, operands in the K-tiled plane
                                 layout (see abq_relayout_planes); tile tuples with NSTAGE = 4 */
    ABQ_STRATEGY_FP6 = 7,     /* FP6 (E2M3) MFMA 32x32x64 at twice the int8 rate, exact for operands
                                 of at most 4 bits unsigned / 5 bits signed (see
                                 abq_relayout_planes_fp6); tile tuples with NSTAGE = 5, MMA 32x32x64 */
    ABQ_STRATEGY_DECODE_TILED = 8 /* int8 MFMA 16x16x64 for decode-sized M on operands that are both in the
                                 K-tiled layout (widths 2, 4 or 8 bits; unsigned 8-bit codes with their row
                                 sums set, abq_gemm_set_row_sums; other widths as padded records,
                                 abq_relayout_planes_padded):
                                 nothing is expanded or transposed inside the kernel; tile tuples with
                                 NSTAGE = 6.  A state with M <= 16 whose operands are both declared
                                 ABQ_LAYOUT_TILED moves here by itself, and so does one of up to 128 rows
                                 where the library estimates this kernel, run over blocks of 16 rows, ahead
                                 of the prefill kernel's smallest tile (narrow pairs, few blocks); with
                                 group scales of 128 and M <= 16 it runs this strategy's group-scale variant
                                 (zero points, fused SiLU gate) */
} abq_strategy;

/* Parses "AqBMMA_8x2xtrue_1x48x512_8x24x128_8x8x128_4" (an optional _InitFn/_ExecFn suffix is
 * accepted).  *is_wmma is set for the AqBWMMA family (engine/mma_any/aq_wmma_op.h), which maps
 * to the same kernels.  Replaces the named globals declared by AQ_DECL_FUN
 * (engine/common/base.h:159-166). */
abq_status abq_parse_kernel_name(const char *name, abq_tile_config *cfg, int *is_wmma);
/* Inverse of the above; writes at most n bytes including the terminator. */
abq_status abq_format_kernel_name(const abq_tile_config *cfg, int is_wmma, char *buf, size_t n);

/* Number of native gfx950 tile configurations for a bit combination, and the i-th one.
 * This is the search space the autotuner walks (the role of engine/gen_kernel.cpp:24-157). */
int abq_native_config_count(int x_bits, int w_bits, int is_signed);
abq_status abq_native_config_get(int x_bits, int w_bits, int is_signed, int index,
                                 abq_tile_config *cfg);

/* ---------------------------------------------------------------------------------------
 * GEMM
 * ------------------------------------------------------------------------------------- */
typedef struct abq_dim3 {
    unsigned x, y, z;
} abq_dim3;

typedef enum abq_out_kind {
    ABQ_OUT_I32 = 0,        /* int32 D (engine/mma_any/aq_bmma_kernel.h:485-580)                 */
    ABQ_OUT_F16_TENSOR = 1, /* fp16 D = half(acc) * C[0], C one fp16 on the device
                               (FT abqgemm/mma_any/aq_bmma_kernel.h:479,516-519)               */
    ABQ_OUT_F16_SCALED = 2, /* fp16 D = acc * x_scale[m] * w_scale[n] (fp32 math), per-token
                               and per-channel scales; see abq_gemm_set_scales                 */
    ABQ_OUT_F16_TENSOR_F32SCALE = 3 /* as ABQ_OUT_F16_TENSOR, but C points to one float on the
                               device, converted to fp16 first: what the FT wrapper means when it
                               hands `const float* scale_out` to the kernel
                               (abq_gemm_wrapper.cu:125-126)                                   */
} abq_out_kind;

/* Launch state, the POD returned by the reference's InitFn (AqBMMAOpState,
 * engine/mma_any/aq_bmma_op.h:19-32).  Caller owned; init fills it, exec only reads it. */
typedef struct abq_gemm_state {
    size_t shared_mem_size;
    abq_dim3 grid_dim;
    abq_dim3 block_dim;
    int init_success;
    /* Argument_t */
    int M, N, K;
    const uint32_t *X;
    const uint32_t *W;
    const void *C;
    void *D;
    int bias;
    /* resolved configuration */
    abq_tile_config cfg;
    int strategy; /* abq_strategy actually used */
    int variant;  /* index into the strategy's kernel table */
    int out_kind; /* abq_out_kind */
    /* optional dequantization operands (ABQ_OUT_F16_SCALED) */
    const float *x_scale;  /* [M] per token            */
    const float *w_scale;  /* [N] or [N][K/group_size] */
    int group_size;        /* 0 = per channel          */
    int reserved[5];       /* [0] popcount kernels: log2 of the lanes per weight row; [1] see
                              abq_gemm_set_dynamic_f16_activations; [2], [3] see abq_gemm_set_value_bits; [4] bits 0, 1 see
                              abq_gemm_set_biased_records, bit 2 abq_gemm_set_padded_activations */
    /* K-tiled operands (ABQ_STRATEGY_TILED) */
    int x_layout, w_layout;  /* abq_layout of X and W as handed to init                    */
    int auto_chosen;         /* 1 if the tile was the library's choice                     */
    void *workspace;         /* caller-owned device scratch for the layout conversions     */
    size_t workspace_bytes;
    /* zero points of the group-scale path, see abq_gemm_set_zero_points */
    const float *x_zero;
    const float *w_zero;
    const int32_t *x_group_sums;
    const float *w_zero_term;
    int act;                 /* abq_activation fused into the epilogue */
    const float *x_pack_scale; /* x_layout == ABQ_LAYOUT_F16: the static quantisation scale, see abq_gemm_set_f16_activations */
    /* row sums of unsigned operands, see abq_gemm_set_row_sums */
    const int32_t *x_row_sums;
    const int32_t *w_row_sums;
} abq_gemm_state;

/* Replaces AqBMMAInitFn / AqBWMMAInitFn (engine/mma_any/aq_bmma_op.h:141-147,163 and
 * aq_wmma_op.h) and AqBMMAOp::initialize (:76-115).  cfg may be NULL (library chooses).
 * x_bits / w_bits / is_signed are read from cfg when given, else from the three ints.
 * `bias` must be 0 (the reference asserts the same, aq_bmma_op.h:79).
 * On failure state->init_success is 0 and the status says why. */
abq_status abq_gemm_init(const abq_tile_config *cfg, int x_bits, int w_bits, int is_signed,
                         const uint32_t *X, const uint32_t *W, int M, int N, int K, void *D,
                         const void *C, int bias, int out_kind, abq_gemm_state *state);

/* Attaches per-token / per-channel scales to an initialised state (ABQ_OUT_F16_SCALED).
 * New behaviour with respect to the reference kernels; the semantics follow
 * algorithm/quantize/quantizer.py:111-179 (scale per row of X, per row of W). */
abq_status abq_gemm_set_scales(abq_gemm_state *state, const float *x_scale, const float *w_scale,
                               int group_size);
/* group_size 0: w_scale is [N] and D = acc * x_scale[m] * w_scale[n].
 * group_size 64 or 128: w_scale is [N][K/group_size] (the reference reshapes W to
 * [-1, group_size] before calibrating, quantizer.py:151-156) and
 *     D[m][n] = x_scale[m] * sum_g w_scale[n][g] * (sum_{k in g} x[m][k] * w[n][k]).
 * Four kernels carry group scales, and a state whose tile was the library's choice is moved to the one that
 * fits: M <= 16 on plane operands -> the group-scale variant of ABQ_STRATEGY_DECODE (64 or 128); M <= 16 with both
 * operands ABQ_LAYOUT_TILED, groups of 128 and widths of 2, 4 or 8 bits -> that of ABQ_STRATEGY_DECODE_TILED (whichever
 * of abq_gemm_set_scales and abq_gemm_set_operand_layout comes first); FP6 operands -> ABQ_STRATEGY_FP6 (128
 * only); everything else -> ABQ_STRATEGY_TILED (and needs the workspace / layouts of that strategy).  A state
 * pinned to a tile tuple of another strategy, or 8-bit unsigned operands, return ABQ_ERR_UNSUPPORTED.  If the call
 * fails the state is left as it was. */

/* Zero points for a state with group scales (asymmetric quantisation, quantizer.py:120-128:
 * x ~ scale * (code - zero)).  Codes are the integers in the bit planes, read with the
 * state's signedness; a caller holding unsigned codes u in [0, 2^n) and zero point z may store
 * u - 2^(n-1) in signed planes and pass z - 2^(n-1).
 *   w_zero       [N][K/group_size]  weight zero points, or NULL
 *   x_group_sums [M][K/group_size]  sums of the activation codes per group; required with w_zero
 *                                   (abq_quant_pack_f16 writes them)
 *   x_zero       [M]                activation zero points, or NULL
 *   w_zero_term  [N]                required with x_zero (abq_weight_zero_term computes it once
 *                                   per weight matrix)
 *     D[m][n] = x_scale[m] * ( sum_g w_scale[n][g] * (acc_g - w_zero[n][g] * x_group_sums[m][g])
 *                              - x_zero[m] * w_zero_term[n] ). */
abq_status abq_gemm_set_zero_points(abq_gemm_state *state, const float *x_zero, const float *w_zero,
                                    const int32_t *x_group_sums, const float *w_zero_term);

/* Activation fused into the dequantising epilogue of a state with group scales.
 * ABQ_ACT_SILU_GATE serves the gate / up pair of a LLaMA MLP (the reference runs them as two GEMMs
 * followed by an elementwise kernel, FfnLayer.cc:341-374,575-577): W holds both matrices
 * interleaved in blocks of 16 rows (gate rows 16b..16b+15, then up rows 16b..16b+15), N counts the
 * rows of both and must be a multiple of 32, and D is [M][N/2]:
 *     D[m][16 b + c] = silu(out[m][32 b + c]) * out[m][32 b + 16 + c],
 * `out` being what the epilogue would have written without the activation. */
typedef enum abq_activation {
    ABQ_ACT_NONE = 0,
    ABQ_ACT_SILU_GATE = 1
} abq_activation;
abq_status abq_gemm_set_activation(abq_gemm_state *state, int act);

/* w_zero_term[n] = sum_g w_scale[n][g] * (sum_{k in g} w[n][k] - group_size * w_zero[n][g]),
 * from weight planes in the reference layout.  w_zero may be NULL (all zero). */
abq_status abq_weight_zero_term(const uint32_t *w_planes, int n, int k, int bits, int is_signed,
                                const float *w_scale, const float *w_zero, int group_size,
                                float *w_zero_term, void *stream);

/* Per-token dynamic quantisation of fp16 activations [rows][k] fused with bit-plane packing:
 * the device-side counterpart of the reference's per_token_dynamic_calibration + fake_quant
 * rounding (algorithm/quantize/quantizer.py:111-179) followed by pack.  Writes signed codes
 * (two's complement planes, `bits` planes) in the layout asked for, scale[rows], and
 * optionally zero[rows] (NULL allowed when symmetric) and group_sums[rows][k/group_size]
 * (NULL, or group_size 64 / 128).
 *   symmetric != 0: scale = clamp(absmax / (2^(bits-1) - 1), 1e-5, 1e4), zero = 0
 *   symmetric == 0: scale = clamp((max - min) / (2^bits - 1), 1e-5, 1e4),
 *                   zp = round(clamp(-min / scale, -1e4, 1e4)), stored code = u - 2^(bits-1),
 *                   zero = zp - 2^(bits-1)
 * fp32 arithmetic, round half to even.  2 <= bits <= 8 (<= 5 for ABQ_LAYOUT_FP6), k % 128 == 0. */
abq_status abq_quant_pack_f16(const void *x_f16, int rows, int k, int bits, int symmetric, int layout,
                              uint32_t *planes, float *scale, float *zero, int32_t *group_sums,
                              int group_size, void *stream);

/* ---------------------------------------------------------------------------------------
 * K-tiled plane layout (no counterpart in the reference; its kernels only exist for M <= 8).
 *
 * The prefill kernels (ABQ_STRATEGY_TILED) read the same bits in the order
 *     tiled[kt][row][plane][4 words],   kt = K / 128 tiles,
 * so that the rows of a workgroup tile are contiguous and every cache line fetched is used in
 * full.  Same size as the reference layout.  Weights are static: convert them once with
 * abq_relayout_planes and declare the layout with abq_gemm_set_operand_layout.  Operands left in
 * the reference layout are converted inside abq_gemm_exec on every call into the caller's
 * workspace (abq_gemm_set_workspace): activations always are unless the caller packs them
 * tiled, weights only if they were not prepared.
 * ------------------------------------------------------------------------------------- */
typedef enum abq_layout {
    ABQ_LAYOUT_PLANES = 0, /* the reference's wire format */
    ABQ_LAYOUT_TILED = 1,
    ABQ_LAYOUT_FP6 = 2,    /* records of 6-bit sign-magnitude codes, see below */
    ABQ_LAYOUT_F16 = 3     /* activations only, set by abq_gemm_set_f16_activations: X is the fp16 matrix itself */
} abq_layout;

/* bytes of a packed operand in either layout */
size_t abq_planes_bytes(int rows, int k, int bits);

/* planes [bits][rows][k/32] -> tiled [k/128][rows][bits][4]; k % 128 == 0. */
abq_status abq_relayout_planes(const uint32_t *planes, uint32_t *tiled, int rows, int k, int bits,
                               void *stream);

/* abq_pack_f16 (pack_half of the reference, abq_gemm_wrapper.cu:29-69: same values, same scale) writing the
 * K-tiled layout directly: bit for bit what abq_relayout_planes makes of abq_pack_f16's planes, without the
 * second pass.  bits <= 8, k % 128 == 0. */
abq_status abq_pack_f16_tiled(const void *in_f16, const float *scale_dev, uint32_t *tiled, int rows, int k, int bits,
                              void *stream);
/* The same values written as FP6 records (abq_relayout_planes_fp6's layout; bits <= 5 signed, <= 4 unsigned): bit for
 * bit what abq_relayout_planes_fp6 makes of abq_pack_f16's planes, i.e. the low `bits` bits of the truncated product
 * read as the code they are (the reference does not clamp, pack_half, abq_gemm_wrapper.cu:42-49).  What
 * ABQGEMMWrapper::gemm packs its activations into when the weight was also prepared as FP6 records. */
abq_status abq_pack_f16_fp6(const void *in_f16, const float *scale_dev, uint32_t *records, int rows, int k, int bits,
                            int is_signed, void *stream);

/* FP6 records (no counterpart in the reference): the operand format of ABQ_STRATEGY_FP6.
 * CDNA4's matrix cores multiply 6-bit floats (E2M3) at twice their int8 rate, and an integer of
 * magnitude <= 16 written as sign and magnitude is an E2M3 number (value / 8), so operands that
 * are unsigned of at most 4 bits or signed of at most 5 bits run there with bit-exact int32
 * results as long as max|x| * max|w| * K < 2^24 (fp32 accumulation of integers).  A record is
 * 24 words per row and K tile of 128 elements: fp6[k/128][rows][24], 3/4 byte per element
 * whatever the bit width.  abq_fp6_eligible tells whether a bit pair and K qualify. */
size_t abq_fp6_bytes(int rows, int k);
int abq_fp6_eligible(int x_bits, int w_bits, int is_signed, int k);

/* Whether a GEMM of this shape whose operands are both K-tiled runs ABQ_STRATEGY_DECODE_TILED when the tile is the
 * library's choice: always up to 16 rows where that kernel is built for the pair (and, with group scales, for
 * groups of 128), and up to 128 rows where the library estimates the kernel, run over blocks of 16 rows, ahead of
 * the prefill kernel.  For callers that hold their weights in several prepared forms and have to pick one before
 * they quantise the activations (ABQGEMMWrapper::gemm_dynamic).  No counterpart in the reference. */
int abq_prepared_decode_pays(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size, int act);
/* planes [bits][rows][k/32] -> fp6 [k/128][rows][24]; bits <= 4, or <= 5 if is_signed. */
abq_status abq_relayout_planes_fp6(const uint32_t *planes, uint32_t *fp6, int rows, int k, int bits,
                                   int is_signed, void *stream);

/* Declares the layout of X and W of an initialised state.  A tiled (FP6) operand moves a state
 * whose tile was the library's choice to ABQ_STRATEGY_TILED (ABQ_STRATEGY_FP6), or, with both operands tiled and
 * M <= 16 (or M <= 128 where the decode kernel over blocks of 16 rows is estimated ahead), to
 * ABQ_STRATEGY_DECODE_TILED where that kernel exists for the pair and epilogue; a state
 * initialised with an explicit tile tuple of another strategy is refused (ABQ_ERR_UNSUPPORTED),
 * and so are a tiled and an FP6 operand together, an FP6 operand with group scales of groups other
 * than 128, and an FP6 operand of a bit pair or K that does not qualify.  A call that is refused leaves the state as
 * it was.  One case changes the pair: signed activations of 3, 5, 6 or 7 bits that stay in planes, above 16 rows,
 * against K-tiled weights of 2, 4 or 8 bits (W2A6): exec converts the activations anyway, so it writes them as records
 * of the next width of one field and the state becomes that pair's (cfg.x_bits = abq_padded_bits, the codes' width
 * kept as by abq_gemm_set_value_bits), which runs the LDS-staged kernel instead of the register-staged one of the odd
 * widths; size the workspace with abq_gemm_workspace_bytes AFTER this call. */
abq_status abq_gemm_set_operand_layout(abq_gemm_state *state, int x_layout, int w_layout);

/* Decode without a packing launch (ABQGEMMWrapper::gemm of the reference packs A and runs the GEMM, two launches,
 * fastertransformer/src/fastertransformer/kernels/abqgemm/abq_gemm_wrapper.cu:79-138; at M = 1 the second costs as
 * much as the first).  On a state that runs ABQ_STRATEGY_DECODE_TILED (M <= 16, prepared weights) with signed
 * 8-bit activations and no group scales, X becomes the fp16 activations [M][K] themselves: every workgroup
 * quantises the rows it multiplies, value = (int)(half(x) * half(scale_dev[0])) as abq_pack_f16 does, into its
 * LDS.  Results are bit for bit those of abq_pack_f16_tiled followed by the same GEMM.  Any other state:
 * ABQ_ERR_UNSUPPORTED, and the caller packs as before. */
abq_status abq_gemm_set_f16_activations(abq_gemm_state *state, const void *x_f16, const float *scale_dev);

/* The group-scale variant of the same: a state that runs ABQ_STRATEGY_DECODE_TILED with group scales of 128 (at most
 * 16 rows, M * K <= 16384, 8-bit signed activations, prepared weights) takes its activations as fp16 [M][K] and
 * quantises them per token inside the kernel, symmetric (symmetric != 0) or with a zero point, with the formulas
 * and the rounding of abq_quant_pack_f16 (bit for bit: the output equals that of the two launches).  The token
 * scales, zero points and group sums never leave the kernel: x_scale given to abq_gemm_set_scales is not read, and
 * abq_gemm_set_zero_points, called after this, takes w_zero (x_group_sums may be NULL) and, for activations with a
 * zero point, w_zero_term (x_zero may be NULL).  One launch instead of two and no memory round trip between them:
 * the quantising launch costs as much as the GEMM at these sizes.  ABQ_ERR_UNSUPPORTED where the kernel or the
 * shape does not qualify (the caller then quantises with abq_quant_pack_f16 as before).  No counterpart in the
 * reference, whose activations are quantised by a kernel of their own (abq_gemm_wrapper.cu:29-69). */
abq_status abq_gemm_set_dynamic_f16_activations(abq_gemm_state *state, const void *x_f16, int symmetric);

/* ---------------------------------------------------------------------------------------
 * Table of measured best tiles (the autotune result)
 *
 * The reference's sweep prints "The best kernel config is ..." (engine/test/test_mma/test_mma.h:21-45,
 * test_mma_w2a8.cu:700) and its authors hard-code that tile in the FT wrapper (abq_gemm_wrapper.cu:105-124).
 * Here engine/test_any_mma --tuning-out appends its best lines to a text file, one entry per line,
 *     <kernel name> <M> <N> <K> <group size> <TOPS>        ('#' starts a comment)
 * the file shipped with the library (engine/tuning_mi355x.txt) is compiled in, and abq_gemm_init(cfg = NULL),
 * abq_gemm_set_operand_layout, abq_gemm_set_scales and abq_gemm_set_workspace look their shape up before they go by
 * the library's rules: among the entries of the same bit pair, signedness, N, K, group size and M bucket (1, 2, 3-4,
 * 5-8, 9-16, 17-32, 33-64, ...) whose tile runs on the layouts the operands are held in, the one with the highest
 * TOPS (entries loaded or added at run time before the compiled-in ones).  The table is the library's only mutable
 * global state; it is guarded by a mutex.
 * ------------------------------------------------------------------------------------- */
/* Reads a file of entries; *entries (may be NULL) receives how many were taken.  ABQ_ERR_INVALID_ARG if the file
 * cannot be read or holds a malformed line (then nothing of it is taken). */
abq_status abq_tuning_load(const char *path, int *entries);
/* Adds one entry: cfg carries bit widths, signedness and the tile tuple. */
abq_status abq_tuning_add(const abq_tile_config *cfg, int M, int N, int K, int group_size, float tops);
/* Forgets the entries loaded or added at run time (the compiled-in ones stay). */
void abq_tuning_clear(void);
/* Switches the compiled-in entries off (0) or back on (1): a harness that measures the rules themselves. */
void abq_tuning_enable_builtin(int on);
/* The entry a state of this shape would be moved to.  layout_mask: bit (1 << abq_layout) set for every layout the
 * weights may be held in (0 = any).  ABQ_ERR_UNSUPPORTED if the table holds nothing for the shape. */
abq_status abq_tuning_lookup(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size, int layout_mask,
                             abq_tile_config *cfg, float *tops);
/* The abq_layout a loader should prepare a weight matrix in for GEMMs of about M rows: the layout of the table's best
 * entry for the shape; without one, FP6 records for pairs that qualify (abq_fp6_eligible) from 257 rows up (1025 for weights of at most 2 bits), K-tiled
 * records otherwise.  (A model that runs prefill and decode on one matrix keeps both where the memory allows.) */
int abq_preferred_weight_layout(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size);
/* The same for a loader that can also write padded records (abq_relayout_planes_padded): *record_bits receives the
 * width of the records to write, w_bits or abq_padded_bits(w_bits).  Weights of 2, 4 or 8 bits: as above.  Weights of
 * 3, 5, 6 or 7 bits run fastest on the kernels of the padded pair at every M, so the answer is that pair's
 * (K-tiled records of the padded width, GEMM initialised with the padded pair and abq_gemm_set_value_bits; or FP6
 * records, which are the same for both widths), except signed 5-bit weights under activations of at most 5 bits
 * above 16 rows, which stay on FP6 records.  No counterpart in the reference. */
int abq_preferred_weight_records(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size, int *record_bits);

/* sums[row] = sum over k of the unsigned codes of a row of an operand in the plane layout ([bits][rows][k/32]).
 * For pairs with an unsigned 8-bit operand: the LDS-staged kernel feeds such an operand to the signed matrix
 * cores as value - 128 and adds 128 x the OTHER operand's row sums to the result (and takes off 2^14 K when both
 * operands are 8 bits wide); it does not gather the sums itself.  Once per weight matrix, beside
 * abq_relayout_planes; once per call for the activations.  No counterpart in the reference, whose binary tensor
 * cores need no such correction (its unsigned instances: engine/test_w4a4_uint_wmma.cu:228-229, FT
 * abqgemm/mma_any/aq_bmma_impl/aq_bmma_w2a8.cu:4-9). */
abq_status abq_row_sums(const uint32_t *planes, int rows, int k, int bits, int32_t *sums, void *stream);

/* Hands the row sums of an unsigned pair's operands to a state (either may be NULL): x_row_sums[M] is read when the
 * weights are 8 bits wide, w_row_sums[N] when the activations are.  abq_gemm_exec on ABQ_STRATEGY_TILED then runs
 * the staged kernel for the tiles it is built for.  Sums that are not set are taken by abq_gemm_exec itself for an
 * operand still in the plane layout if the workspace has the room (abq_gemm_workspace_bytes counts them); when a
 * needed sum is neither set nor to be had, the kernel that gathers the sums inside its K loop runs instead (same
 * tile, same result, slower).  Ignored by signed pairs and by pairs without an 8-bit operand. */
abq_status abq_gemm_set_row_sums(abq_gemm_state *state, const int32_t *x_row_sums, const int32_t *w_row_sums);
/* 1 if abq_gemm_exec on this state, as it stands, runs the kernel that takes the row sums handed in (every needed
 * sum set, or to be had from plane operands into the workspace the state holds), 0 otherwise. */
int abq_gemm_row_sums_ready(const abq_gemm_state *state);

/* Biased records of unsigned W8A8.  abq_relayout_planes_biased writes the K-tiled records of an unsigned 8-bit
 * operand with 128 taken off every code (bit 7 flipped): the byte is then the int8 the signed matrix cores want, and
 * the staged kernel spends nothing on flipping it after every LDS read (W8A8 uint then runs the signed pair's
 * kernel).  abq_gemm_set_biased_records(state, x_biased, w_biased) declares which K-tiled operands of an unsigned
 * W8A8 state are such records: the weights (prepared once, with their row sums set through abq_gemm_set_row_sums),
 * and the activations if the caller prepared them the same way; activations that arrive as planes are converted
 * that way by abq_gemm_exec itself, and their row sums taken, in the workspace.  Only the prefill kernel
 * (ABQ_STRATEGY_TILED) on the tiles the staged kernel is built for reads them; x_biased without w_biased is refused.
 * ABQ_ERR_UNSUPPORTED for any other pair.  No counterpart in the reference. */
abq_status abq_relayout_planes_biased(const uint32_t *planes, uint32_t *tiled, int rows, int k, void *stream);
abq_status abq_gemm_set_biased_records(abq_gemm_state *state, int x_biased, int w_biased);

/* Padded records for the widths made of several fields.  The decode kernel on prepared operands reads records of one
 * field per element (2, 4 or 8 bits).  An operand of 3, 5, 6 or 7 bits is brought to it as records of the next such
 * width, abq_padded_bits(bits) (1, 2 -> 2; 3, 4 -> 4; 5..8 -> 8), the code of every element extended to that width
 * (sign extension for signed codes): the values, and therefore the GEMM, are the same, the records are
 * abq_planes_bytes(rows, k, abq_padded_bits(bits)) long.  The GEMM is then initialised with the padded widths, its
 * operands declared ABQ_LAYOUT_TILED, and (unsigned pairs whose records are 8 bits wide) told through
 * abq_gemm_set_value_bits how many bits the codes really have: 8-bit records of at most 7-bit codes are fed to the
 * matrix cores as they are, while true 8-bit codes need the value - 128 route and its row sums.  For widths of one
 * field the call equals abq_relayout_planes.  No counterpart in the reference (its binary tensor cores take any
 * number of planes; its decode sweep over these widths: engine/test.sh:8-206). */
int abq_padded_bits(int bits);
abq_status abq_relayout_planes_padded(const uint32_t *planes, uint32_t *tiled, int rows, int k, int bits, int is_signed,
                                      void *stream);
/* Weights with group-wise zero points as records that need no zero-point term: every code has its group's zero point
 * taken off, w_zero[row][k / group_size] (a whole number, as the quantiser's rounding leaves it), and the signed
 * differences, one bit wider than the codes, are written as K-tiled records of abq_folded_bits(bits) bits (2 -> 4,
 * 3 -> 4, 4 ... 7 -> 8; 0 for 8: not supported).  A GEMM on them is initialised as the signed pair (x_bits,
 * abq_folded_bits(bits)) with the group scales and WITHOUT weight zero points (abq_gemm_set_zero_points: w_zero and
 * x_group_sums NULL; the activation zero points' w_zero_term stays what abq_weight_zero_term made of the original
 * weights): out = sum_g sx sw[n,g] sum_k x (w - z) is the same number, and the epilogue's zero-point term, 10-20 %
 * of a prefill GEMM with group scales, is gone, for records twice the size of 2-bit weights: a copy for prefill-sized
 * calls where the memory is there.  group_size: a multiple of 32 that divides k (and of 128, or a divisor of it).
 * misfit_dev (may be NULL): a device int the caller has zeroed, set to 1 if a zero point is no whole number or a
 * difference does not fit the records.  No counterpart in the reference (its zero points: quantizer.py:111-132). */
int abq_folded_bits(int bits);
abq_status abq_relayout_planes_folded(const uint32_t *planes, const float *w_zero, int group_size, uint32_t *tiled, int rows, int k,
                                      int bits, int is_signed, int *misfit_dev, void *stream);

/* The same for FP6 records (abq_relayout_planes_fp6's layout, same size): codes of at most 4 bits less whole-number
 * zero points have magnitudes of at most 16 and therefore FP6 codes.  A GEMM on them is initialised like one on
 * abq_relayout_planes_fp6's records, under the pair's own widths, SIGNED (activations that are unsigned codes come as
 * FP6 records too, which hold their values), without weight zero points; exact for K up to 65536.  misfit_dev as
 * above. */
abq_status abq_relayout_planes_fp6_folded(const uint32_t *planes, const float *w_zero, int group_size, uint32_t *fp6, int rows, int k,
                                          int bits, int is_signed, int *misfit_dev, void *stream);

/* Declares that the codes of X (W) use only the low x_value_bits (w_value_bits) of their fields (1 .. the state's
 * widths): see above.  An operand of such a state that is still in the reference plane layout has that many planes,
 * and abq_gemm_exec extends its codes to the records' width while it converts them into the workspace.  This makes
 * padded weight records serve every M: above 16 rows the padded pair's prefill kernels run (the LDS-staged int8
 * kernel for 8-bit records, which the widths of several fields do not have), and an unsigned pair whose codes are
 * narrower than the records on both sides runs the signed pair's kernel of the same tile: such codes are signed codes
 * of the records' width as well, so neither the value - 128 route nor row sums are needed. */
abq_status abq_gemm_set_value_bits(abq_gemm_state *state, int x_value_bits, int w_value_bits);
/* Weights of 3, 5, 6 or 7 bits need no padded copy for decode: the decode kernel on prepared operands reads the
 * records abq_relayout_planes writes (the ones the prefill kernels read), field by field.  Its activations are records
 * of one field; a state whose ACTIVATIONS are 3, 5, 6 or 7 bits wide therefore takes them as padded records
 * (abq_relayout_planes_padded, abq_planes_bytes(M, k, abq_padded_bits(x_bits)) bytes), declared ABQ_LAYOUT_TILED and
 * marked with this call (before or after abq_gemm_set_operand_layout; activations handed over as planes are converted
 * that way by abq_gemm_exec itself, abq_gemm_workspace_bytes counts the padded size).  The state is initialised with
 * the pair's own widths.  Up to 16 rows; ABQ_ERR_UNSUPPORTED where only the prefill kernel could run, which reads
 * records of the activations' own width.  No effect for activations of 2, 4 or 8 bits.  No counterpart in the
 * reference (its decode sweep over these widths: engine/test.sh:8-206). */
abq_status abq_gemm_set_padded_activations(abq_gemm_state *state, int padded);

/* Workspace needed by abq_gemm_exec if the state ran as ABQ_STRATEGY_TILED, ABQ_STRATEGY_DECODE_TILED
 * (ABQ_STRATEGY_FP6) with its current operand layouts: the converted copies of the operands still in
 * the reference layout.  Operands declared K-tiled (FP6 records) count 0, and so do fp16 activations
 * handed to the decode kernel (ABQ_LAYOUT_F16: quantised inside the kernel, nothing is converted). */
size_t abq_gemm_workspace_bytes(const abq_gemm_state *state);

/* Hands a caller-owned device buffer to the state.  If the tile was the library's choice, M > 64
 * (32 for outputs of 8192 columns or more; 16 with group scales) and the buffer is large enough, the
 * state moves to ABQ_STRATEGY_TILED; otherwise it keeps its kernel (which needs no workspace:
 * below those sizes the conversion launch costs more than the LDS-staged kernel gains).  A state on
 * ABQ_STRATEGY_TILED whose weights are K-tiled and whose activations are planes, 17 to 128 rows, moves to
 * ABQ_STRATEGY_DECODE_TILED where that kernel is estimated ahead (either converts the activations into the
 * workspace first; size the buffer with abq_gemm_workspace_bytes before and after: the need does not grow). */
abq_status abq_gemm_set_workspace(abq_gemm_state *state, void *workspace, size_t bytes);

/* Replaces AqBMMAExecFn / AqBWMMAExecFn (engine/mma_any/aq_bmma_op.h:155-161,164): one
 * asynchronous launch on `stream`. */
abq_status abq_gemm_exec(const abq_gemm_state *state, void *stream);

/* No counterpart in the reference.  abq_gemm_exec for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the same launches, with
 * the layout conversions writing into a static device array inside the library instead of a workspace the
 * caller brings (a workspace attached to the state is ignored).  Allocates nothing.  A state whose
 * conversions need more than ABQ_STATIC_WORKSPACE_BYTES is refused with ABQ_ERR_TOO_LARGE and a message
 * on stderr.  All calls on one device share that device's array: calls that may run concurrently on one
 * device (different streams) race on it; order them or use abq_gemm_exec with separate workspaces.  The
 * first call on a device looks the array's address up (hipGetSymbolAddress): make it before a capture. */
#define ABQ_STATIC_WORKSPACE_BYTES (32u << 20)
abq_status abq_gemm_exec_static(const abq_gemm_state *state, void *stream);

/* Replaces launchWmmaAnyKernel (engine/wmma_any/wmma_any.h:18-38, wmma_any.cu:28-87): the
 * first-generation entry point, init + exec in one call, int32 D. */
abq_status abq_gemm_launch(const abq_tile_config *cfg, const uint32_t *X, const uint32_t *W,
                           const void *C, int32_t *D, int bias, int M, int N, int K, void *stream);


#ifdef __cplusplus
}
#endif
#endif /* ABQ_GEMM_H */
