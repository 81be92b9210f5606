// See abq_weight_file.h.
#include "abq_weight_file.h"

#include <math.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>

#include "abq_gemm.h"

static const char kMagic[8] = { 'A', 'B', 'Q', 'W', 'G', 'T', '1', '\0' };

static bool fail(std::string *error, const std::string &what)
{
    if (error)
        *error = what;
    return false;
}

bool abq_quantize_weights(const float *w, uint32_t n, uint32_t k, uint32_t nominal_bits, bool symmetric, uint32_t group_size,
                          ABQWeightBlob *out, std::string *error, bool bit_balance)
{
    if (!w || !out || n == 0 || nominal_bits < (bit_balance ? 1u : 2u) || nominal_bits > 8)
        return fail(error, "bad arguments");
    if (bit_balance && (symmetric || nominal_bits > 2))
        return fail(error, "bit balance applies to asymmetric 1- and 2-bit weights only");
    // with bit balance the unsigned codes run from 0 to 2^bits inclusive: one more plane
    const uint32_t bits = bit_balance ? nominal_bits + 1 : nominal_bits;
    const int levels = bit_balance ? (1 << nominal_bits) : (1 << nominal_bits) - 1; // qmax of the unsigned code
    if (k < 128 || k % 128 != 0)
        return fail(error, "K must be >= 128 and a multiple of 128");
    const uint32_t g = group_size ? group_size : k;
    if (k % g != 0 || g % 32 != 0)
        return fail(error, "group_size must divide K and be a multiple of 32");
    const uint32_t groups = k / g;
    const int half = 1 << (bits - 1);
    memset(&out->info, 0, sizeof(out->info));
    out->info.reserved[0] = bit_balance ? 1u : 0u;
    memcpy(out->info.magic, kMagic, 8);
    out->info.version = 1;
    out->info.n = n;
    out->info.k = k;
    out->info.bits = bits;
    out->info.is_signed = 1;
    out->info.group_size = group_size;
    out->info.has_zero = symmetric ? 0 : 1;
    const size_t kw = k / 32;
    out->planes.assign((size_t)bits * n * kw, 0u);
    out->scale.assign((size_t)n * groups, 0.f);
    out->zero.assign(symmetric ? 0 : (size_t)n * groups, 0.f);
    for (uint32_t r = 0; r < n; ++r) {
        for (uint32_t gi = 0; gi < groups; ++gi) {
            const float *x = w + (size_t)r * k + (size_t)gi * g;
            double mn = x[0], mx = x[0];
            for (uint32_t i = 1; i < g; ++i) {
                mn = std::min(mn, (double)x[i]);
                mx = std::max(mx, (double)x[i]);
            }
            double scale, zp = 0;
            if (symmetric) {
                scale = std::max(fabs(mn), fabs(mx)) / (half - 1);
                scale = std::min(std::max(scale, 1e-5), 1e4);
            } else {
                scale = (mx - mn) / levels;
                scale = std::min(std::max(scale, 1e-5), 1e4);
                zp = nearbyint(std::min(std::max(-mn / scale, -1e4), 1e4));
            }
            out->scale[(size_t)r * groups + gi] = (float)scale;
            if (!symmetric)
                out->zero[(size_t)r * groups + gi] = (float)(zp - half);
            for (uint32_t i = 0; i < g; ++i) {
                double q = nearbyint((double)x[i] / scale); // round half to even, as torch.round
                int code;
                if (symmetric)
                    code = (int)std::min(std::max(q, (double)-half), (double)(half - 1));
                else
                    code = (int)std::min(std::max(q + zp, 0.0), (double)levels) - half;
                const uint32_t e = gi * g + i; // element within the row
                const uint32_t pattern = (uint32_t)code & ((1u << bits) - 1u);
                for (uint32_t b = 0; b < bits; ++b)
                    if ((pattern >> b) & 1u)
                        out->planes[((size_t)b * n + r) * kw + e / 32] |= 1u << (31 - e % 32);
            }
        }
    }
    return true;
}

bool abq_weight_blob_interleave_gate_up(const ABQWeightBlob &gate, const ABQWeightBlob &up, ABQWeightBlob *out,
                                        std::string *error)
{
    const ABQWeightHeader &a = gate.info, &b = up.info;
    if (!out || a.n != b.n || a.k != b.k || a.bits != b.bits || a.is_signed != b.is_signed || a.group_size != b.group_size ||
        a.has_zero != b.has_zero)
        return fail(error, "gate and up blobs do not have the same shape and quantisation");
    if (a.n % 16 != 0)
        return fail(error, "row count must be a multiple of 16");
    const size_t kw = a.k / 32, groups = gate.groups(), n = a.n;
    out->info = a;
    out->info.n = 2 * a.n;
    out->planes.resize(gate.planes.size() * 2);
    out->scale.resize(gate.scale.size() * 2);
    out->zero.resize(gate.zero.size() * 2);
    for (size_t row = 0; row < 2 * n; ++row) {
        const size_t blk = row / 32, within = row % 32;
        const ABQWeightBlob &src = within < 16 ? gate : up;
        const size_t srow = blk * 16 + within % 16;
        for (uint32_t p = 0; p < a.bits; ++p)
            memcpy(&out->planes[((size_t)p * 2 * n + row) * kw], &src.planes[((size_t)p * n + srow) * kw], kw * 4);
        memcpy(&out->scale[row * groups], &src.scale[srow * groups], groups * 4);
        if (a.has_zero)
            memcpy(&out->zero[row * groups], &src.zero[srow * groups], groups * 4);
    }
    return true;
}

static bool check_header(const ABQWeightHeader &h, std::string *error)
{
    if (memcmp(h.magic, kMagic, 8) != 0 || h.version != 1)
        return fail(error, "not an ABQWGT1 file");
    if (h.n == 0 || h.bits < 1 || h.bits > 8 || h.k < 128 || h.k % 128 != 0)
        return fail(error, "bad shape in header");
    if (h.group_size && (h.k % h.group_size != 0))
        return fail(error, "bad group size in header");
    return true;
}

bool abq_weight_file_write(const std::string &path, const ABQWeightBlob &blob, std::string *error)
{
    if (!check_header(blob.info, error))
        return false;
    const size_t plane_words = (size_t)blob.info.bits * blob.info.n * (blob.info.k / 32);
    const size_t ns = (size_t)blob.info.n * blob.groups();
    if (blob.planes.size() != plane_words || blob.scale.size() != ns || blob.zero.size() != (blob.info.has_zero ? ns : 0))
        return fail(error, "blob sizes do not match its header");
    FILE *f = fopen(path.c_str(), "wb");
    if (!f)
        return fail(error, "cannot open " + path + " for writing");
    bool ok = fwrite(&blob.info, sizeof(blob.info), 1, f) == 1 &&
              fwrite(blob.planes.data(), 4, plane_words, f) == plane_words &&
              fwrite(blob.scale.data(), 4, ns, f) == ns &&
              (!blob.info.has_zero || fwrite(blob.zero.data(), 4, ns, f) == ns);
    ok = (fclose(f) == 0) && ok;
    return ok ? true : fail(error, "short write to " + path);
}

bool abq_weight_file_read(const std::string &path, ABQWeightBlob *blob, std::string *error)
{
    if (!blob)
        return fail(error, "bad arguments");
    FILE *f = fopen(path.c_str(), "rb");
    if (!f)
        return fail(error, "cannot open " + path);
    bool ok = fread(&blob->info, sizeof(blob->info), 1, f) == 1 && check_header(blob->info, error);
    if (ok) {
        const size_t plane_words = (size_t)blob->info.bits * blob->info.n * (blob->info.k / 32);
        const size_t ns = (size_t)blob->info.n * blob->groups();
        blob->planes.resize(plane_words);
        blob->scale.resize(ns);
        blob->zero.resize(blob->info.has_zero ? ns : 0);
        ok = fread(blob->planes.data(), 4, plane_words, f) == plane_words && fread(blob->scale.data(), 4, ns, f) == ns &&
             (!blob->info.has_zero || fread(blob->zero.data(), 4, ns, f) == ns);
        if (ok && fgetc(f) != EOF)
            ok = false; // trailing bytes: not a file this code wrote
        if (!ok)
            fail(error, "truncated or oversized file " + path);
    } else if (error && error->empty()) {
        *error = "cannot read header of " + path;
    }
    fclose(f);
    return ok;
}

bool abq_weight_file_write_ft_bin(const std::string &path, const ABQWeightBlob &blob, std::string *error)
{
    FILE *f = fopen(path.c_str(), "wb");
    if (!f)
        return fail(error, "cannot open " + path + " for writing");
    bool ok = fwrite(blob.planes.data(), 4, blob.planes.size(), f) == blob.planes.size();
    ok = (fclose(f) == 0) && ok;
    return ok ? true : fail(error, "short write to " + path);
}

ABQDeviceWeight::~ABQDeviceWeight() { release(); }

void ABQDeviceWeight::release()
{
    for (void *p : { (void *)planes_, (void *)tiled_, (void *)fp6_, (void *)padded_, (void *)folded_, (void *)scale_, (void *)zero_,
                     (void *)zero_term_ })
        if (p)
            (void)hipFree(p);
    planes_ = tiled_ = fp6_ = padded_ = folded_ = nullptr;
    fp6_is_folded_ = false;
    scale_ = zero_ = zero_term_ = nullptr;
}

bool ABQDeviceWeight::load(const ABQWeightBlob &blob, hipStream_t stream, std::string *error)
{
    release();
    if (!check_header(blob.info, error))
        return false;
    info_ = blob.info;
    const size_t plane_bytes = blob.planes.size() * 4, ns = blob.scale.size();
    auto hip_ok = [&](hipError_t e, const char *what) {
        if (e == hipSuccess)
            return true;
        fail(error, std::string(what) + ": " + hipGetErrorString(e));
        return false;
    };
    if (!hip_ok(hipMalloc(&planes_, plane_bytes), "hipMalloc planes") || !hip_ok(hipMalloc(&tiled_, plane_bytes), "hipMalloc tiled") ||
        !hip_ok(hipMalloc(&scale_, ns * 4), "hipMalloc scale") || !hip_ok(hipMalloc(&zero_term_, (size_t)info_.n * 4), "hipMalloc zero_term"))
        return false;
    if (info_.has_zero && !hip_ok(hipMalloc(&zero_, ns * 4), "hipMalloc zero"))
        return false;
    if (!hip_ok(hipMemcpyAsync(planes_, blob.planes.data(), plane_bytes, hipMemcpyHostToDevice, stream), "upload planes") ||
        !hip_ok(hipMemcpyAsync(scale_, blob.scale.data(), ns * 4, hipMemcpyHostToDevice, stream), "upload scale"))
        return false;
    if (info_.has_zero && !hip_ok(hipMemcpyAsync(zero_, blob.zero.data(), ns * 4, hipMemcpyHostToDevice, stream), "upload zero"))
        return false;
    abq_status rc = abq_relayout_planes(planes_, tiled_, (int)info_.n, (int)info_.k, (int)info_.bits, stream);
    if (rc == ABQ_OK && (info_.group_size == 64 || info_.group_size == 128))
        rc = abq_weight_zero_term(planes_, (int)info_.n, (int)info_.k, (int)info_.bits, (int)info_.is_signed, scale_, zero_,
                                  (int)info_.group_size, zero_term_, stream);
    // FP6 records for the FP6 matrix-core route (groups of 128; codes of magnitude at most 16)
    if (rc == ABQ_OK && info_.group_size == 128 && info_.bits <= (info_.is_signed ? 5u : 4u)) {
        if (!hip_ok(hipMalloc(&fp6_, abq_fp6_bytes((int)info_.n, (int)info_.k)), "hipMalloc fp6"))
            return false;
        rc = abq_relayout_planes_fp6(planes_, fp6_, (int)info_.n, (int)info_.k, (int)info_.bits, (int)info_.is_signed, stream);
        // with whole-number zero points (and at most 4 bits) the same records hold code - zero point instead
        if (rc == ABQ_OK && info_.has_zero && info_.bits <= 4u) {
            int *misfit = nullptr, host_misfit = 1;
            uint32_t *folded = nullptr;
            if (!hip_ok(hipMalloc(&folded, abq_fp6_bytes((int)info_.n, (int)info_.k)), "hipMalloc fp6 folded") ||
                !hip_ok(hipMalloc(&misfit, sizeof(int)), "hipMalloc flag") || !hip_ok(hipMemsetAsync(misfit, 0, sizeof(int), stream), "clear flag"))
                return false;
            const abq_status frc = abq_relayout_planes_fp6_folded(planes_, zero_, 128, folded, (int)info_.n, (int)info_.k, (int)info_.bits,
                                                                  (int)info_.is_signed, misfit, stream);
            const bool copied = hip_ok(hipMemcpyAsync(&host_misfit, misfit, sizeof(int), hipMemcpyDeviceToHost, stream), "read flag") &&
                                hip_ok(hipStreamSynchronize(stream), "synchronise");
            (void)hipFree(misfit);
            if (!copied) {
                (void)hipFree(folded);
                return false;
            }
            if (frc == ABQ_OK && !host_misfit) {
                (void)hipFree(fp6_);
                fp6_ = folded;
                fp6_is_folded_ = true;
            } else {
                (void)hipFree(folded);
            }
        }
    }
    // padded records for the widths of several fields: the kernels of the next single-field width read those
    if (rc == ABQ_OK && abq_padded_bits((int)info_.bits) != (int)info_.bits) {
        if (!hip_ok(hipMalloc(&padded_, abq_planes_bytes((int)info_.n, (int)info_.k, abq_padded_bits((int)info_.bits))), "hipMalloc padded"))
            return false;
        rc = abq_relayout_planes_padded(planes_, padded_, (int)info_.n, (int)info_.k, (int)info_.bits, (int)info_.is_signed, stream);
    }
    // zero points folded into the records, for prefill-sized calls: kept only if every zero point is a whole number
    // and the differences fit (the quantiser's rounded zero points do)
    if (rc == ABQ_OK && info_.has_zero && (info_.group_size == 64 || info_.group_size == 128) && abq_folded_bits((int)info_.bits) != 0) {
        int *misfit = nullptr, host_misfit = 1;
        if (!hip_ok(hipMalloc(&folded_, abq_planes_bytes((int)info_.n, (int)info_.k, abq_folded_bits((int)info_.bits))), "hipMalloc folded") ||
            !hip_ok(hipMalloc(&misfit, sizeof(int)), "hipMalloc flag") || !hip_ok(hipMemsetAsync(misfit, 0, sizeof(int), stream), "clear flag"))
            return false;
        rc = abq_relayout_planes_folded(planes_, zero_, (int)info_.group_size, folded_, (int)info_.n, (int)info_.k, (int)info_.bits,
                                        (int)info_.is_signed, misfit, stream);
        const bool copied = hip_ok(hipMemcpyAsync(&host_misfit, misfit, sizeof(int), hipMemcpyDeviceToHost, stream), "read flag") &&
                            hip_ok(hipStreamSynchronize(stream), "synchronise");
        (void)hipFree(misfit);
        if (!copied)
            return false;
        if (rc != ABQ_OK || host_misfit) { // such weights keep the zero-point term
            (void)hipFree(folded_);
            folded_ = nullptr;
            rc = rc == ABQ_ERR_UNSUPPORTED ? ABQ_OK : rc;
        } else if (padded_ && abq_folded_bits((int)info_.bits) == abq_padded_bits((int)info_.bits)) {
            (void)hipFree(padded_); // records of the same width without the zero points: gemm_dynamic runs every call on the folded ones
            padded_ = nullptr;
        }
    }
    if (rc != ABQ_OK)
        return fail(error, std::string("weight preparation failed: ") + abq_status_string(rc));
    return hip_ok(hipStreamSynchronize(stream), "synchronise");
}

ABQGroupedWeight ABQDeviceWeight::grouped() const
{
    return ABQGroupedWeight{ reinterpret_cast<const int *>(tiled_), scale_, zero_, zero_term_, (int)info_.group_size,
                             reinterpret_cast<const int *>(planes_), fp6_is_folded_ ? nullptr : reinterpret_cast<const int *>(fp6_),
                             reinterpret_cast<const int *>(padded_), reinterpret_cast<const int *>(folded_),
                             fp6_is_folded_ ? reinterpret_cast<const int *>(fp6_) : nullptr };
}
