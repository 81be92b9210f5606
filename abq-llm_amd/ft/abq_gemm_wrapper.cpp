// See abq_gemm_wrapper.h.  Follows the decision table of the reference's
// ABQGEMMWrapper::gemm (abq_gemm_wrapper.cu:79-138): quantise + pack A, check K, pick a kernel,
// init, check initSuccess, exec.
#include "abq_gemm_wrapper.h"

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <unordered_map>

#include "abq_gemm.h"

namespace {

struct PreparedWeight {
    int N, K, bits;
    bool ready;              // false while prepare_weight is still converting (the entry reserves the pointer)
    uint32_t fingerprint[16]; // the first 64 bytes of the prepared records, for verify_prepared
};

// FP6 records registered for a weight pointer (prepare_weight_fp6): a second copy for prefill-sized calls
struct Fp6Weight {
    const int *records;
    int N, K, bits;
    bool is_signed;
};

std::unordered_map<const void *, Fp6Weight> &fp6_table()
{
    static std::unordered_map<const void *, Fp6Weight> table;
    return table;
}

std::mutex g_prepared_mutex;

std::unordered_map<const void *, PreparedWeight> &prepared_table()
{
    static std::unordered_map<const void *, PreparedWeight> table;
    return table;
}

bool find_prepared(const void *B, PreparedWeight *out)
{
    std::lock_guard<std::mutex> lock(g_prepared_mutex);
    const auto it = prepared_table().find(B);
    if (it == prepared_table().end() || !it->second.ready)
        return false;
    *out = it->second;
    return true;
}

// ABQ_VERIFY_PREPARED=1 in the environment: every gemm() on a prepared weight first compares the weight's first
// record with what prepare_weight left there (a device read and a synchronisation per call: for debugging a
// loader that frees or refills weight buffers without release_weight, not for production).
bool verify_on_every_call()
{
    static const bool on = [] {
        const char *v = getenv("ABQ_VERIFY_PREPARED");
        return v && v[0] == '1';
    }();
    return on;
}

} // namespace

size_t ABQGEMMWrapper::prepared_weight_bytes(int N, int K, int W_BITS) { return abq_planes_bytes(N, K, W_BITS); }

bool ABQGEMMWrapper::prepare_weight(int *B, int N, int K, int W_BITS, int *scratch, hipStream_t stream)
{
    if (!B || !scratch || N <= 0 || K < 128 || K % 128 != 0 || W_BITS < 1 || W_BITS > 8) {
        printf("[ABQ][Error] prepare_weight: bad argument (N, K, bits = %d, %d, %d)\n", N, K, W_BITS);
        return false;
    }
    {
        // check and insert in one critical section: of two threads that prepare the same B one is refused; the
        // entry is not ready (gemm() does not see it) until the records are in place
        std::lock_guard<std::mutex> lock(g_prepared_mutex);
        if (prepared_table().count(B)) {
            printf("[ABQ][Error] prepare_weight: %p is prepared already\n", (void *)B);
            return false;
        }
        prepared_table()[B] = PreparedWeight{ N, K, W_BITS, false, { 0 } };
    }
    auto fail = [&](const char *what) {
        printf("[ABQ][Error] prepare_weight failed: %s\n", what);
        std::lock_guard<std::mutex> lock(g_prepared_mutex);
        prepared_table().erase(B);
        return false;
    };
    const abq_status rc = abq_relayout_planes(reinterpret_cast<const uint32_t *>(B), reinterpret_cast<uint32_t *>(scratch),
                                              N, K, W_BITS, stream);
    if (rc != ABQ_OK)
        return fail(abq_status_string(rc));
    hipError_t e = hipMemcpyAsync(B, scratch, abq_planes_bytes(N, K, W_BITS), hipMemcpyDeviceToDevice, stream);
    if (e != hipSuccess)
        return fail(hipGetErrorString(e));
    // the first record's bytes as they now are (one small read and a synchronisation, once per weight matrix)
    PreparedWeight entry{ N, K, W_BITS, true, { 0 } };
    const size_t nfp = abq_planes_bytes(N, K, W_BITS) < sizeof entry.fingerprint ? abq_planes_bytes(N, K, W_BITS) : sizeof entry.fingerprint;
    e = hipMemcpyAsync(entry.fingerprint, B, nfp, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess)
        e = hipStreamSynchronize(stream);
    if (e != hipSuccess)
        return fail(hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_prepared_mutex);
    prepared_table()[B] = entry;
    return true;
}

bool ABQGEMMWrapper::verify_prepared(const int *B, hipStream_t stream)
{
    PreparedWeight w;
    if (!find_prepared(B, &w))
        return false;
    uint32_t now[16] = { 0 };
    const size_t nfp = abq_planes_bytes(w.N, w.K, w.bits) < sizeof now ? abq_planes_bytes(w.N, w.K, w.bits) : sizeof now;
    if (hipMemcpyAsync(now, B, nfp, hipMemcpyDeviceToHost, stream) != hipSuccess || hipStreamSynchronize(stream) != hipSuccess)
        return false;
    return memcmp(now, w.fingerprint, nfp) == 0;
}

size_t ABQGEMMWrapper::fp6_weight_bytes(int N, int K) { return abq_fp6_bytes(N, K); }

bool ABQGEMMWrapper::prepare_weight_fp6(const int *B, int N, int K, int W_BITS, bool SIGNED, int *records, hipStream_t stream)
{
    if (!B || !records || N <= 0 || K < 128 || K % 128 != 0 || W_BITS < 1 || W_BITS > (SIGNED ? 5 : 4)) {
        printf("[ABQ][Error] prepare_weight_fp6: bad argument (N, K, bits = %d, %d, %d)\n", N, K, W_BITS);
        return false;
    }
    if (is_prepared(B)) { // its planes are gone
        printf("[ABQ][Error] prepare_weight_fp6: %p has been rewritten by prepare_weight already; call this one first\n", (const void *)B);
        return false;
    }
    const abq_status rc = abq_relayout_planes_fp6(reinterpret_cast<const uint32_t *>(B), reinterpret_cast<uint32_t *>(records), N, K,
                                                  W_BITS, SIGNED ? 1 : 0, stream);
    if (rc != ABQ_OK) {
        printf("[ABQ][Error] prepare_weight_fp6 failed: %s\n", abq_status_string(rc));
        return false;
    }
    std::lock_guard<std::mutex> lock(g_prepared_mutex);
    fp6_table()[B] = Fp6Weight{ records, N, K, W_BITS, SIGNED };
    return true;
}

void ABQGEMMWrapper::release_weight(const int *B)
{
    std::lock_guard<std::mutex> lock(g_prepared_mutex);
    prepared_table().erase(B);
    fp6_table().erase(B);
}

bool ABQGEMMWrapper::is_prepared(const int *B)
{
    PreparedWeight w;
    return find_prepared(B, &w);
}

ABQGEMMWrapper::ABQGEMMWrapper(int X_BITS, int W_BITS, bool SIGNED) : x_bits_(X_BITS), w_bits_(W_BITS), signed_(SIGNED) {}

ABQGEMMWrapper::~ABQGEMMWrapper() {}

void ABQGEMMWrapper::pack(const _Float16 *in_data, const float *scale, int *packed_data, int M, int K, int BIT,
                          hipStream_t stream)
{
    const abq_status rc = abq_pack_f16(in_data, scale, reinterpret_cast<uint32_t *>(packed_data), M, K, BIT, stream);
    if (rc != ABQ_OK)
        printf("[ABQ][Error] pack failed: %s\n", abq_status_string(rc));
}

void ABQGEMMWrapper::pack(const int *in_data, int *packed_data, int M, int K, int BIT, hipStream_t stream)
{
    const abq_status rc = abq_pack_i32(in_data, reinterpret_cast<uint32_t *>(packed_data), M, K, BIT, stream);
    if (rc != ABQ_OK)
        printf("[ABQ][Error] pack failed: %s\n", abq_status_string(rc));
}

void ABQGEMMWrapper::gemm(const int M, const int N, const int K, const _Float16 *A, const int *B, const _Float16 *C,
                          _Float16 *D, const float *scale, const float *scale_inter, const float *scale_out, bool bias,
                          char *abq_gemm_workspace, size_t abq_gemm_ws_bytes, hipStream_t stream)
{
    (void)C;
    (void)scale_inter;
    if (K < 128 || K % 128 != 0) {
        printf("[ABQ][Error] unsupport K = %d\n", K);
        return;
    }
    if (abq_gemm_ws_bytes < (size_t)x_bits_ * M * K / 8) {
        printf("[ABQ][Error] workspace too small: %zu bytes for M,K,bits = %d,%d,%d\n", abq_gemm_ws_bytes, M, K, x_bits_);
        return;
    }
    // Prefill-sized calls on a pair that qualifies for the FP6 matrix cores, when the loader registered FP6 records
    // for this weight and the workspace holds the activations as such records (6 bits per element): twice the
    // matrix-core rate of the int8 route, and nothing to unpack.
    {
        Fp6Weight f6{};
        bool have = false;
        {
            std::lock_guard<std::mutex> lock(g_prepared_mutex);
            const auto it = fp6_table().find(B);
            if (it != fp6_table().end()) {
                f6 = it->second;
                have = true;
            }
        }
        if (have && M > 16 && f6.N == N && f6.K == K && f6.bits == w_bits_ && f6.is_signed == signed_ &&
            abq_fp6_eligible(x_bits_, w_bits_, signed_ ? 1 : 0, K) && abq_gemm_ws_bytes >= abq_fp6_bytes(M, K) &&
            abq_preferred_weight_layout(x_bits_, w_bits_, signed_ ? 1 : 0, M, N, K, 0) == ABQ_LAYOUT_FP6) {
            abq_gemm_state st;
            abq_status rc = abq_pack_f16_fp6(A, scale, reinterpret_cast<uint32_t *>(abq_gemm_workspace), M, K, x_bits_, signed_ ? 1 : 0, stream);
            if (rc == ABQ_OK)
                rc = abq_gemm_init(nullptr, x_bits_, w_bits_, signed_ ? 1 : 0, reinterpret_cast<const uint32_t *>(abq_gemm_workspace),
                                   reinterpret_cast<const uint32_t *>(f6.records), M, N, K, D, scale_out, bias ? 1 : 0,
                                   ABQ_OUT_F16_TENSOR_F32SCALE, &st);
            if (rc == ABQ_OK)
                rc = abq_gemm_set_operand_layout(&st, ABQ_LAYOUT_FP6, ABQ_LAYOUT_FP6);
            if (rc == ABQ_OK && st.init_success) {
                const abq_status ex = abq_gemm_exec(&st, stream);
                if (ex != ABQ_OK)
                    printf("[ABQ][Error] launch failed: %s\n", abq_status_string(ex));
                return;
            }
            // (anything the FP6 route refuses: the routes below)
        }
    }
    PreparedWeight prepared;
    const bool tiled = find_prepared(B, &prepared);
    if (tiled && verify_on_every_call() && !verify_prepared(B, stream)) {
        printf("[ABQ][Error] %p is in the table of prepared weights but no longer holds the prepared records "
               "(freed or refilled without release_weight?)\n", (const void *)B);
        return;
    }
    if (tiled && (prepared.N != N || prepared.K != K || prepared.bits != w_bits_)) {
        printf("[ABQ][Error] weight prepared as N, K, bits = %d, %d, %d, called with %d, %d, %d\n", prepared.N, prepared.K,
               prepared.bits, N, K, w_bits_);
        return;
    }
    abq_gemm_state state;
    abq_status rc = abq_gemm_init(nullptr, x_bits_, w_bits_, signed_ ? 1 : 0,
                                  reinterpret_cast<const uint32_t *>(abq_gemm_workspace),
                                  reinterpret_cast<const uint32_t *>(B), M, N, K, D, scale_out, bias ? 1 : 0,
                                  ABQ_OUT_F16_TENSOR_F32SCALE, &state);
    if (rc == ABQ_ERR_UNSUPPORTED) {
        printf("[ABQ][Error] unsupport w%da%d\n", w_bits_, x_bits_);
        return;
    }
    if (rc == ABQ_OK && tiled)
        rc = abq_gemm_set_operand_layout(&state, ABQ_LAYOUT_TILED, ABQ_LAYOUT_TILED);
    if (rc != ABQ_OK || !state.init_success) {
        printf("[ABQ][Error] return due to unsuccessful initialization.\n");
        return;
    }
    // quant + packing; for a prepared weight straight into the layout its kernels read, or, for decode-sized calls
    // with 8-bit activations, inside the GEMM kernel itself (one launch instead of two)
    // (where a workgroup quantises its rows in one pass, M * K <= 32768, and the workgroups that all repeat that are
    // few enough: 3.9 against 5.2 us at M = 1 and 5.0 against 5.5 at M = 8 on 4096 x 4096, 5.8 against 6.5 at M = 1 on
    // 11008 x 4096; on wider outputs, or from M = 4 on outputs beyond 4096, the packing launch is the cheaper way:
    // 22016 x 4096 at M = 1 8.6 against 9.4 us, 11008 x 4096 at M = 8 6.9 against 10.2)
    const bool in_kernel = (long)M * K <= 32768 && (N <= 4096 || (M == 1 && N <= 12288));
    if (tiled && in_kernel && abq_gemm_set_f16_activations(&state, A, scale) == ABQ_OK) {
        // nothing to pack
    } else if (tiled) {
        const abq_status prc = abq_pack_f16_tiled(A, scale, reinterpret_cast<uint32_t *>(abq_gemm_workspace), M, K, x_bits_, stream);
        if (prc != ABQ_OK) {
            printf("[ABQ][Error] pack failed: %s\n", abq_status_string(prc));
            return;
        }
    } else {
        pack(A, scale, reinterpret_cast<int *>(abq_gemm_workspace), M, K, x_bits_, stream);
    }
    const abq_status ex = abq_gemm_exec(&state, stream);
    if (ex != ABQ_OK)
        printf("[ABQ][Error] launch failed: %s\n", abq_status_string(ex));
}

void ABQGEMMWrapper::gemm_scaled(const int M, const int N, const int K, const int *X_packed, const int *B, _Float16 *D,
                                 const float *x_scale, const float *w_scale, hipStream_t stream)
{
    if (K < 128 || K % 128 != 0) {
        printf("[ABQ][Error] unsupport K = %d\n", K);
        return;
    }
    if (is_prepared(B)) { // its words are K-tiled records now: read as planes they would give wrong numbers silently
        printf("[ABQ][Error] gemm_scaled takes weight planes; %p has been rewritten by prepare_weight\n", (const void *)B);
        return;
    }
    abq_gemm_state state;
    abq_status rc = abq_gemm_init(nullptr, x_bits_, w_bits_, signed_ ? 1 : 0, reinterpret_cast<const uint32_t *>(X_packed),
                                  reinterpret_cast<const uint32_t *>(B), M, N, K, D, nullptr, 0, ABQ_OUT_F16_SCALED, &state);
    if (rc == ABQ_OK)
        rc = abq_gemm_set_scales(&state, x_scale, w_scale, 0);
    if (rc != ABQ_OK || !state.init_success) {
        printf("[ABQ][Error] return due to unsuccessful initialization.\n");
        return;
    }
    const abq_status ex = abq_gemm_exec(&state, stream);
    if (ex != ABQ_OK)
        printf("[ABQ][Error] launch failed: %s\n", abq_status_string(ex));
}

// workspace: activation planes | scale[M] | zero[M] | group sums [M][K/group_size]
size_t ABQGEMMWrapper::dynamic_workspace_bytes(int M, int K, int group_size) const
{
    return activation_bytes(M, K) + (size_t)M * 8 + (size_t)M * (K / group_size) * 4;
}

// packed activations of a call: x_bits per element, or 6 where they may be written as FP6 records
size_t ABQGEMMWrapper::activation_bytes(int M, int K) const
{
    const int bits = abq_fp6_eligible(x_bits_, w_bits_, signed_ ? 1 : 0, K) ? 6 : x_bits_;
    return ((size_t)bits * M * K / 8 + 255) / 256 * 256;
}

void ABQGEMMWrapper::gemm_dynamic(const int M, const int N, const int K, const _Float16 *A, const ABQGroupedWeight &W_given,
                                  _Float16 *D, bool x_symmetric, char *abq_gemm_workspace, size_t abq_gemm_ws_bytes,
                                  hipStream_t stream, bool silu_gate)
{
    // Weights of 3, 5, 6 or 7 bits whose folded records are as wide as their padded ones: the folded records take the
    // padded records' place in every call, and the weights have no zero points any more (W3A8 with groups of 128 at one
    // token: 3.8 / 6.7 / 7.3 us against 4.0 / 7.3 / 8.1 on padded records with zero points)
    ABQGroupedWeight W = W_given;
    if (W.records_folded && abq_native_config_count(x_bits_, abq_folded_bits(w_bits_), 1) <= 0)
        W.records_folded = nullptr; // (no kernels for the activations' width against the folded records')
    if (W.records_folded && W.zero && abq_padded_bits(w_bits_) != w_bits_ && abq_folded_bits(w_bits_) == abq_padded_bits(w_bits_)) {
        W.records_padded = W.records_folded;
        W.records_folded = nullptr;
        W.zero = nullptr;
    }
    // (FP6 records with the zero points folded in stand for the plain ones on the FP6 route)
    const bool fp6_folded = W.records_fp6_folded != nullptr && W.zero != nullptr && w_bits_ <= 4;
    const int *const records_fp6 = fp6_folded ? W.records_fp6_folded : W.records_fp6;
    if (K < 128 || K % 128 != 0) {
        printf("[ABQ][Error] unsupport K = %d\n", K);
        return;
    }
    if (!signed_ || (W.group_size != 64 && W.group_size != 128) || (!x_symmetric && !W.zero_term)) {
        printf("[ABQ][Error] unsupport dynamic quantisation setup\n");
        return;
    }
    if (W.planes && is_prepared(W.planes)) {
        printf("[ABQ][Error] ABQGroupedWeight::planes %p has been rewritten by prepare_weight: hand it over as planes_tiled\n",
               (const void *)W.planes);
        return;
    }
    if (abq_gemm_ws_bytes < dynamic_workspace_bytes(M, K, W.group_size)) {
        printf("[ABQ][Error] workspace too small: %zu bytes for M,K,bits = %d,%d,%d\n", abq_gemm_ws_bytes, M, K, x_bits_);
        return;
    }
    const size_t planes_bytes = activation_bytes(M, K);
    uint32_t *planes = reinterpret_cast<uint32_t *>(abq_gemm_workspace);
    float *x_scale = reinterpret_cast<float *>(abq_gemm_workspace + planes_bytes);
    float *x_zero = x_scale + M;
    int32_t *sums = reinterpret_cast<int32_t *>(x_zero + M);
    // at most 16 rows (and small batches above that where the library estimates it ahead): the decode kernel on
    // prepared operands where it is built for the pair (widths of 2, 4 or 8 bits, groups of 128; the library moves
    // the state there once both layouts are declared), else the decode kernel on plane operands if the caller kept
    // the planes; otherwise the tiled kernel on the prefill layout
    // (weights of several fields: as padded records, on the padded pair's kernel, the codes' own width declared)
    const int w_rec_bits = abq_padded_bits(w_bits_);
    const bool w_padded = w_rec_bits != w_bits_;
    const uint32_t *w_records = reinterpret_cast<const uint32_t *>(w_padded ? W.records_padded : W.planes_tiled);
    const bool decode_prepared = w_records != nullptr &&
                                 abq_prepared_decode_pays(x_bits_, w_rec_bits, 1, M, N, K, W.group_size, silu_gate ? 1 : 0) != 0;
    // (if the expanded activations fit the decode kernel's LDS: partial tiles, group sums, M padded rows)
    const bool decode = !decode_prepared && M <= 16 && W.planes != nullptr &&
                        (silu_gate ? 32 : 16) * 1024 + (size_t)64 * (K / W.group_size) + 128 + (size_t)M * ((K + 511) / 512 * 512 + 16) <= 160 * 1024;
    // (FP6 records where the library prefers them for the shape: from 257 rows unless a measured entry says otherwise; below,
    // the int8 route's small tiles are ahead, W4A4 with groups of 128 at 128 x 4096 x 4096 13.7 against 19.7 us.  A weight
    // that has no other records runs on them at every size.)
    const bool fp6 = !decode && !decode_prepared && records_fp6 != nullptr && W.group_size == 128 && abq_fp6_eligible(x_bits_, w_bits_, 1, K) &&
                     (w_records == nullptr || abq_preferred_weight_layout(x_bits_, w_bits_, 1, M, N, K, 128) == ABQ_LAYOUT_FP6);
    const int layout = decode ? ABQ_LAYOUT_PLANES : fp6 ? ABQ_LAYOUT_FP6 : ABQ_LAYOUT_TILED;
    abq_status rc;
    abq_gemm_state state;
    // the smallest calls on the prepared-operand decode kernel: the kernel quantises the rows itself (one launch
    // instead of two; the quantising launch costs as much as the GEMM at these sizes), same result bit for bit
    // (one token, or several on outputs of at most 4096 columns: every workgroup repeats the quantisation, which on
    // the wide linears costs more than the launch from two tokens on: QKV of LLaMA-7B at two tokens 11.6 against
    // 10.1 us, at four 18.0 against 10.7; 4096 x 4096 at four tokens 8.1 against 8.6)
    if (decode_prepared && M <= 16 && (size_t)M * K <= 16384 && (M == 1 || N <= 4096)) {
        rc = abq_gemm_init(nullptr, x_bits_, w_rec_bits, 1, planes, w_records, M, N, K, D, nullptr, 0, ABQ_OUT_F16_SCALED, &state);
        if (rc == ABQ_OK && w_padded)
            rc = abq_gemm_set_value_bits(&state, x_bits_, w_bits_);
        if (rc == ABQ_OK)
            rc = abq_gemm_set_operand_layout(&state, ABQ_LAYOUT_TILED, ABQ_LAYOUT_TILED);
        if (rc == ABQ_OK)
            rc = abq_gemm_set_scales(&state, x_scale /* not read */, W.scale, W.group_size);
        if (rc == ABQ_OK && silu_gate)
            rc = abq_gemm_set_activation(&state, ABQ_ACT_SILU_GATE);
        if (rc == ABQ_OK)
            rc = abq_gemm_set_dynamic_f16_activations(&state, A, x_symmetric ? 1 : 0);
        if (rc == ABQ_OK && (W.zero || !x_symmetric))
            rc = abq_gemm_set_zero_points(&state, nullptr, W.zero, nullptr, x_symmetric ? nullptr : W.zero_term);
        if (rc == ABQ_OK && state.init_success) {
            const abq_status ex = abq_gemm_exec(&state, stream);
            if (ex != ABQ_OK)
                printf("[ABQ][Error] launch failed: %s\n", abq_status_string(ex));
            return;
        }
        // (a pair or shape that kernel does not take: the two launches below)
    }
    rc = abq_quant_pack_f16(A, M, K, x_bits_, x_symmetric ? 1 : 0, layout, planes, x_scale, x_zero,
                            sums, W.group_size, stream);
    if (rc != ABQ_OK) {
        printf("[ABQ][Error] pack failed: %s\n", abq_status_string(rc));
        return;
    }
    // (padded records serve every M: above the decode sizes the padded pair's LDS-staged prefill kernel reads them,
    // which the widths of several fields do not have: W3A8 with groups of 128 at 1024 tokens 1.3-1.7 times faster)
    const bool on_padded = w_padded && W.records_padded != nullptr && !decode && !fp6;
    // (prefill-sized calls on weights whose zero points were folded into the records: no zero-point term)
    const bool on_folded = W.records_folded != nullptr && W.zero != nullptr && !decode && !decode_prepared && !fp6 && M > 16 &&
                           abq_folded_bits(w_bits_) != 0;
    if (!decode && !fp6 && !on_padded && !on_folded && !W.planes_tiled) {
        printf("[ABQ][Error] ABQGroupedWeight::planes_tiled is needed for M,N,K = %d,%d,%d\n", M, N, K);
        return;
    }
    rc = abq_gemm_init(nullptr, x_bits_, on_folded ? abq_folded_bits(w_bits_) : on_padded ? w_rec_bits : w_bits_, 1, planes,
                       decode ? reinterpret_cast<const uint32_t *>(W.planes) : fp6 ? reinterpret_cast<const uint32_t *>(records_fp6)
                       : on_folded ? reinterpret_cast<const uint32_t *>(W.records_folded)
                       : on_padded ? w_records : reinterpret_cast<const uint32_t *>(W.planes_tiled), M, N, K,
                       D, nullptr, 0, ABQ_OUT_F16_SCALED, &state);
    if (rc == ABQ_OK && on_padded && !on_folded)
        rc = abq_gemm_set_value_bits(&state, x_bits_, w_bits_);
    if (rc == ABQ_OK && !decode)
        rc = abq_gemm_set_operand_layout(&state, layout, layout);
    if (rc == ABQ_OK)
        rc = abq_gemm_set_scales(&state, x_scale, W.scale, W.group_size);
    if (rc == ABQ_OK && (on_folded || (fp6 && fp6_folded))) {
        if (!x_symmetric)
            rc = abq_gemm_set_zero_points(&state, x_zero, nullptr, nullptr, W.zero_term);
    } else if (rc == ABQ_OK && (W.zero || !x_symmetric)) {
        rc = abq_gemm_set_zero_points(&state, x_symmetric ? nullptr : x_zero, W.zero, sums, W.zero_term);
    }
    if (rc == ABQ_OK && silu_gate)
        rc = abq_gemm_set_activation(&state, ABQ_ACT_SILU_GATE);
    if (rc == ABQ_ERR_UNSUPPORTED) {
        printf("[ABQ][Error] unsupport w%da%d\n", w_bits_, x_bits_);
        return;
    }
    if (rc != ABQ_OK || !state.init_success) {
        printf("[ABQ][Error] return due to unsuccessful initialization.\n");
        return;
    }
    const abq_status ex = abq_gemm_exec(&state, stream);
    if (ex != ABQ_OK)
        printf("[ABQ][Error] launch failed: %s\n", abq_status_string(ex));
}
