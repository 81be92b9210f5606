// Packed weight files and their device-side preparation.
//
// The reference's FasterTransformer build reads the mode-5 weights of a linear layer as a raw
// dump of the bit planes (LlamaDecoderLayerWeight.cc:377-400 of the reference: a tensor of
// w_bits * K * N / 16 fp16-sized elements per matrix, no header) and leaves the scales as
// "TODO: Load scales" (:401).  This file format carries the same plane bytes after a 64-byte
// header, followed by the scales and zero points the quantiser produced, so one file holds all
// a dequantising GEMM needs; write_ft_bin() emits the headerless plane dump for the reference
// loader.
//
// Layout (little endian):
//   header   64 bytes  (struct ABQWeightHeader)
//   planes   bits * n * k / 8 bytes   planes[b][row][k/32] uint32, element e of a 32-group at bit 31-e
//   scale    float32 [n][groups]      groups = k / group_size, or 1 when group_size == 0
//   zero     float32 [n][groups]      only if has_zero; in units of the signed codes in the planes
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "abq_gemm_wrapper.h"

struct ABQWeightHeader {
    char magic[8]; // "ABQWGT1\0"
    uint32_t version;
    uint32_t n, k;
    uint32_t bits;
    uint32_t is_signed;
    uint32_t group_size; // 0: one scale per output channel
    uint32_t has_zero;
    uint32_t reserved[7];
};
static_assert(sizeof(ABQWeightHeader) == 64, "header is 64 bytes");

struct ABQWeightBlob {
    ABQWeightHeader info;
    std::vector<uint32_t> planes;
    std::vector<float> scale;
    std::vector<float> zero;
    size_t groups() const { return info.group_size ? info.k / info.group_size : 1; }
};

// Quantises a row-major fp32 matrix w[n][k] as the reference's weight quantiser does with
// per_channel_axes = [0] and group_size (algorithm/quantize/quantizer.py:149-179, the plain
// 2^bits - 1 level range): asymmetric codes u in [0, 2^bits) with zero point zp per (row, group),
// stored as signed codes u - 2^(bits-1) with zero = zp - 2^(bits-1); symmetric: signed codes in
// [-2^(bits-1), 2^(bits-1)-1], no zero points.  group_size 0 = one group per row.
// bit_balance (asymmetric 1- and 2-bit weights only): the reference's default at those widths
// (quantizer.py:66-68,169-171): the range is widened by one level, qmax = 2^bits and scale = range / 2^bits, so a
// 2-bit weight takes the five values u in [0, 4].  Five levels do not fit two planes: the codes are stored with
// bits + 1 planes (info.bits = bits + 1, info.reserved[0] = 1) as u - 2^bits with zero = zp - 2^bits, and the GEMM
// runs as a (bits + 1)-bit weight.
bool abq_quantize_weights(const float *w, uint32_t n, uint32_t k, uint32_t bits, bool symmetric, uint32_t group_size,
                          ABQWeightBlob *out, std::string *error, bool bit_balance = false);

// The gate and up projections of one MLP as a single matrix for the fused SiLU-gate epilogue
// (abq_gemm_set_activation): blocks of 16 gate rows followed by their 16 up rows; planes, scales
// and zero points are interleaved alike.  Both blobs must agree in everything but their values,
// and their row count must be a multiple of 16.
bool abq_weight_blob_interleave_gate_up(const ABQWeightBlob &gate, const ABQWeightBlob &up, ABQWeightBlob *out,
                                        std::string *error);

bool abq_weight_file_write(const std::string &path, const ABQWeightBlob &blob, std::string *error);
bool abq_weight_file_read(const std::string &path, ABQWeightBlob *blob, std::string *error);
// headerless plane dump: what LlamaDecoderLayerWeight::loadModel reads for int8_mode 5
bool abq_weight_file_write_ft_bin(const std::string &path, const ABQWeightBlob &blob, std::string *error);

// A weight matrix resident on the device, ready for both kernel families: the planes as they
// are (decode kernels), the prefill layout, scales, zero points and the zero-point term; for the
// widths the kernels read fastest in another form (FP6 records, padded records) that form as well.
class ABQDeviceWeight {
public:
    ABQDeviceWeight() = default;
    ~ABQDeviceWeight();
    ABQDeviceWeight(const ABQDeviceWeight &) = delete;
    ABQDeviceWeight &operator=(const ABQDeviceWeight &) = delete;

    // Uploads the blob and runs the one-time conversions on `stream`; false (with a message) on
    // any HIP or library error.  The stream is synchronised before returning.
    bool load(const ABQWeightBlob &blob, hipStream_t stream, std::string *error);
    void release();

    const int *planes() const { return reinterpret_cast<const int *>(planes_); }
    const ABQWeightHeader &info() const { return info_; }
    // operand of ABQGEMMWrapper::gemm_dynamic (group_size 64 / 128 only)
    ABQGroupedWeight grouped() const;

private:
    ABQWeightHeader info_{};
    uint32_t *planes_ = nullptr, *tiled_ = nullptr, *fp6_ = nullptr; // fp6_: only for groups of 128 and at most 5 (4 unsigned) bits
    uint32_t *padded_ = nullptr;                                     // only for 3, 5, 6, 7 bits: records of the next width of one field
    uint32_t *folded_ = nullptr;                                     // only with whole-number zero points: records of code - zero point
    bool fp6_is_folded_ = false;                                     // fp6_ holds code - zero point as well
    float *scale_ = nullptr, *zero_ = nullptr, *zero_term_ = nullptr;
};
