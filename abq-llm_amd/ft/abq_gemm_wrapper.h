// ABQGEMMWrapper: the class the FasterTransformer LLaMA layers call when int8_mode == 5
// (reference: fastertransformer/src/fastertransformer/kernels/abqgemm/abq_gemm_wrapper.h:6-32;
// call sites FfnLayer.cc:341-374,489-505, DecoderSelfAttentionLayer.cc:605-621,746-761,
// GptContextAttentionLayer.cc:150-166,519-535).  Same constructor and method signatures with
// hipStream_t / _Float16 in place of cudaStream_t / half.
//
// Behaviour kept: activation quantisation value = (int)(half(x) * half(scale[0])) with no
// rounding and no clamp; K must be >= 128 and a multiple of 128; failures print
// "[ABQ][Error] ..." and return.  Behaviour changed on purpose:
//  * every bit combination the library has kernels for is accepted, not only W2A8, and the tile
//    is the library's choice for (M, N, K) instead of the two hard-coded tiles;
//  * scale_out[0] is read as the float it is (the reference reinterprets the pointer as half*
//    and reads the low 16 bits of the float, abq_gemm_wrapper.cu:126);
//  * the workspace size is checked.
// prepare_weight() is new: a loader calls it once per weight matrix; gemm() then runs the kernels built for
// the prepared (K-tiled) layout, for prefill and decode, with unchanged call sites.
// gemm_scaled() is new: per-token activation scales and per-channel weight scales.
// gemm_dynamic() is new: per-token dynamic activation quantisation on the device, group-wise
// weight scales and zero points (the quantiser semantics of algorithm/quantize/quantizer.py).
#pragma once
#include <hip/hip_runtime_api.h>
#include <stddef.h>

// One prepared weight matrix for gemm_dynamic(): device pointers, owned by the caller.
struct ABQGroupedWeight {
    const int *planes_tiled;  // K-tiled planes [K/128][N][w_bits][4] (abq_relayout_planes)
    const float *scale;       // [N][K/group_size]
    const float *zero;        // [N][K/group_size] in units of (signed) weight codes, or nullptr
    const float *zero_term;   // [N] from abq_weight_zero_term; needed for asymmetric activations
    int group_size;           // 64 or 128
    const int *planes;        // the same weights in the reference plane layout [w_bits][N][K/32], or nullptr;
                              // with it, calls of at most 16 rows run the decode kernel on plane operands where
                              // the one on prepared operands does not exist (widths other than 2, 4, 8 bits, groups
                              // of 64); for those that have it, planes_tiled serves every M
    const int *records_fp6;   // the same weights as FP6 records (abq_relayout_planes_fp6), or nullptr; with it,
                              // groups of 128 and a bit pair that qualifies (abq_fp6_eligible, e.g. W4A4), calls of
                              // more than 16 rows run on the FP6 matrix cores
    const int *records_padded; // weights of 3, 5, 6 or 7 bits (e.g. the reference's bit-balanced 2-bit weights, three
                              // planes): the same weights as records of the next single-field width
                              // (abq_relayout_planes_padded), or nullptr; with it, every call runs the padded
                              // pair's kernels on them: the prepared-operand decode kernel instead of the one on plane
                              // operands, the LDS-staged prefill kernel instead of the register-staged one of the
                              // odd widths; planes_tiled may then be nullptr
    const int *records_folded; // weights with whole-number zero points, at most 7 bits: the same weights as records of
                              // code - zero point (abq_relayout_planes_folded; twice the bytes of 2-bit weights), or
                              // nullptr; with it, prefill-sized calls (those that leave the decode kernels) run on
                              // them without the zero-point term, 3-19 % faster (most at K = 11008); for weights of
                              // 3, 5, 6, 7 bits they are as wide as the padded records and serve every call in their
                              // place
    const int *records_fp6_folded; // the FP6 records with the zero points folded in (abq_relayout_planes_fp6_folded; weights
                              // of at most 4 bits), or nullptr; same size as records_fp6 and used in their place: the FP6
                              // route without the zero-point term (QKV of LLaMA-7B at 16384 tokens, W4A4: 10 % faster)
};

class ABQGEMMWrapper {
private:
    int x_bits_;
    int w_bits_;
    bool signed_;

public:
    ABQGEMMWrapper(int X_BITS, int W_BITS, bool SIGNED);
    ~ABQGEMMWrapper();

    void pack(const int *in_data, int *packed_data, int M, int K, int BIT, hipStream_t stream);
    void pack(const _Float16 *in_data, const float *scale, int *packed_data, int M, int K, int BIT,
              hipStream_t stream);
    // One-time weight preparation for gemm() (no counterpart in the reference, whose kernels stop at M = 8; belongs
    // after the loader's reads of the plane files, LlamaDecoderLayerWeight.cc:377-400).  Rewrites the W_BITS planes at
    // B, [W_BITS][N][K/32] device words, in place as K-tiled records (same size) through `scratch`, device memory
    // of prepared_weight_bytes(N, K, W_BITS) that may be freed or reused once `stream` has passed this call, and
    // enters B into a process-wide table.  Every later gemm() of any wrapper whose B is this pointer packs its
    // activations into the same layout and runs the LDS-staged prefill kernel (M > 16) or the decode kernel on
    // prepared operands (M <= 16, and small batches above that where the library estimates it ahead) with no
    // conversion inside the call; a B that was never prepared keeps the plane
    // kernels.  gemm_scaled() and ABQGroupedWeight::planes refuse a B that has been prepared (its words are records
    // now).  Returns false (after "[ABQ][Error] ...") on a bad argument, a failed launch, or a B that is prepared already
    // (check and entry are one critical section: of two threads preparing one B one is refused).  release_weight()
    // takes B out of the table and MUST be called before the memory is freed or refilled: the table goes by the
    // pointer, and a buffer re-allocated at the same address would be read as records.  What the library can do
    // about that without reading device memory in every call: prepare_weight keeps the first 64 bytes of the
    // records (one synchronisation per weight matrix at load time), verify_prepared() compares them with what B
    // holds now (a loader or a test calls it after it has moved weights around), and with ABQ_VERIFY_PREPARED=1 in the
    // environment every gemm() on a prepared weight does so first (one device read and synchronisation per call).
    static size_t prepared_weight_bytes(int N, int K, int W_BITS);
    static bool prepare_weight(int *B, int N, int K, int W_BITS, int *scratch, hipStream_t stream);
    static void release_weight(const int *B);
    static bool is_prepared(const int *B);
    static bool verify_prepared(const int *B, hipStream_t stream);
    // A second copy of a weight matrix for prefill-sized calls on pairs that qualify for the FP6 matrix cores
    // (abq_fp6_eligible: at most 5 bits signed, 4 unsigned, e.g. W4A4): FP6 records of fp6_weight_bytes(N, K) bytes,
    // written to caller-owned `records` from the planes at B and entered into a table under B.  Call it BEFORE
    // prepare_weight (which rewrites the planes).  gemm() on B with more than 16 rows then packs its activations
    // as FP6 records as well (workspace of at least 0.75 M K bytes) and runs the FP6 kernel where
    // abq_preferred_weight_layout names that layout for the shape (the table of measured tiles, else from 65 rows
    // up); every other call keeps the routes of prepare_weight.  release_weight(B) forgets both.
    static size_t fp6_weight_bytes(int N, int K);
    static bool prepare_weight_fp6(const int *B, int N, int K, int W_BITS, bool SIGNED, int *records, hipStream_t stream);

    // A: fp16 activations [M][K]; B: packed weight planes [w_bits][N][K/32]; C unused;
    // D: fp16 [M][N]; scale: activation quantisation scale (1 float, device);
    // scale_inter unused; scale_out: output scale (1 float, device);
    // abq_gemm_workspace: at least X_BITS * M * K / 8 bytes of device memory.
    void gemm(const int M, const int N, const int K, const _Float16 *A, const int *B, const _Float16 *C,
              _Float16 *D, const float *scale, const float *scale_inter, const float *scale_out, bool bias,
              char *abq_gemm_workspace, size_t abq_gemm_ws_bytes, hipStream_t stream);
    // D[m][n] = acc[m][n] * x_scale[m] * w_scale[n]; X given as already packed planes.
    void gemm_scaled(const int M, const int N, const int K, const int *X_packed, const int *B, _Float16 *D,
                     const float *x_scale, const float *w_scale, hipStream_t stream);
    // A: fp16 activations [M][K], quantised per token to X_BITS signed codes inside the call
    // (symmetric, or asymmetric with a zero point); D: fp16 [M][N].  The wrapper must have been
    // constructed with SIGNED = true.  Workspace: dynamic_workspace_bytes(M, K, group_size).
    // silu_gate: W holds a gate / up pair interleaved in blocks of 16 rows (abq_weight_blob_interleave_gate_up),
    // N counts the rows of both and D is [M][N/2] = silu(gate) * up: the two GEMMs and the elementwise
    // kernel of the reference's gated MLP (FfnLayer.cc:341-374,575-577) in one launch.
    // The smallest calls (one token, or up to 16 rows on outputs of at most 4096 columns; M * K <= 16384, 8-bit
    // activations, groups of 128, a pair the prepared-operand decode kernel is built for) are ONE launch: that kernel
    // quantises the rows itself, the
    // workspace is not written, the output is the same bit for bit.
    void gemm_dynamic(const int M, const int N, const int K, const _Float16 *A, const ABQGroupedWeight &W,
                      _Float16 *D, bool x_symmetric, char *abq_gemm_workspace, size_t abq_gemm_ws_bytes,
                      hipStream_t stream, bool silu_gate = false);
    size_t dynamic_workspace_bytes(int M, int K, int group_size) const;
    // the packed activations' share of it (x_bits per element; 6 where the bit pair qualifies for FP6 records)
    size_t activation_bytes(int M, int K) const;
};
