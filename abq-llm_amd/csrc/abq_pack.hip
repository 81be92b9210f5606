// Bit-plane packing kernels.
//
// Replace pack / pack4 (engine/common/pack.cu:18-64 of the reference) and pack_int / pack_half
// (fastertransformer/src/fastertransformer/kernels/abqgemm/abq_gemm_wrapper.cu:9-54).
// Output layout is the reference's: planes[b][r][j], element e of a 32-group at bit 31-e.
//
// The reference launches one thread per output word per plane, so its input is re-read once
// per plane.  Here a lane reads 8 consecutive elements once (32 bytes of int32 or 16 bytes of
// fp16), turns them into one byte per plane with an 8x8 bit transpose, and the four lanes of
// a quad assemble the bytes into one word per plane with DPP moves.  Input bytes are read
// once, every load is 16 bytes wide and consecutive lanes touch consecutive memory.
#include <climits>
#include "abq_kernels.h"
#include "abq_quant.h"

namespace abq {

// OR across the 4 lanes of a quad (all lanes end with the result).
__device__ __forceinline__ uint32_t quad_or(uint32_t v)
{
    v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true); // quad_perm [1,0,3,2]
    v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true); // quad_perm [2,3,0,1]
    return v;
}

// Emits the plane words of one 32-element group; the quad's lane q holds elements 8q..8q+7.
__device__ __forceinline__ void emit_planes(const int (&v)[8], uint32_t *planes, size_t plane_words,
                                            size_t word_idx, int bits, int quad_lane, bool active)
{
    for (int base = 0; base < bits; base += 8) {
        int vs[8];
#pragma unroll
        for (int c = 0; c < 8; ++c)
            vs[c] = active ? (int)((uint32_t)v[c] >> base) : 0;
        const uint64_t bytes = eight_values_to_plane_bytes(vs);
        const int nb = min(8, bits - base);
        for (int b = 0; b < nb; ++b) {
            uint32_t word = (uint32_t)((bytes >> (8 * b)) & 0xFFu) << (24 - 8 * quad_lane);
            word = quad_or(word);
            if (active && quad_lane == 0)
                planes[(size_t)(base + b) * plane_words + word_idx] = word;
        }
    }
}

__global__ __launch_bounds__(256) void pack_i32_kernel(const int4 *__restrict__ in,
                                                       uint32_t *__restrict__ planes,
                                                       size_t n_units, int bits)
{
    const size_t plane_words = n_units / 4;
    // n_units is a multiple of 4 and the stride a multiple of 256, so a quad is active as one.
    const size_t rounded = (n_units + 255) / 256 * 256;
    for (size_t t = (size_t)blockIdx.x * 256 + threadIdx.x; t < rounded; t += (size_t)gridDim.x * 256) {
        const bool active = t < n_units;
        int v[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
        if (active) {
            const int4 lo = in[2 * t], hi = in[2 * t + 1];
            v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
            v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
        }
        emit_planes(v, planes, plane_words, t / 4, bits, (int)(t & 3), active);
    }
}

__global__ __launch_bounds__(256) void pack_f16_kernel(const uint4 *__restrict__ in,
                                                       const float *__restrict__ scale,
                                                       uint32_t *__restrict__ planes,
                                                       size_t n_units, int bits)
{
    const size_t plane_words = n_units / 4;
    const _Float16 hs = (_Float16)scale[0];
    const size_t rounded = (n_units + 255) / 256 * 256;
    for (size_t t = (size_t)blockIdx.x * 256 + threadIdx.x; t < rounded; t += (size_t)gridDim.x * 256) {
        const bool active = t < n_units;
        int v[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
        if (active) {
            union {
                uint4 u;
                _Float16 h[8];
            } raw;
            raw.u = in[t];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const _Float16 p = raw.h[c] * hs; // fp16 product, rounded to nearest even
                v[c] = (int)p;                    // truncation
            }
        }
        emit_planes(v, planes, plane_words, t / 4, bits, (int)(t & 3), active);
    }
}

__global__ __launch_bounds__(256) void pack_u4_kernel(const uint4 *__restrict__ in,
                                                      uint32_t *__restrict__ planes, size_t n_words,
                                                      int bits)
{
    for (size_t t = (size_t)blockIdx.x * 256 + threadIdx.x; t < n_words; t += (size_t)gridDim.x * 256) {
        const uint4 v = in[t];
        for (int b = 0; b < bits; ++b) {
            // For b >= 4 the reference's shifts reach into the neighbouring nibble
            // (pack.cu:28 shifts the whole word); the helper does the same.
            const uint32_t word = (nibble_word_plane_byte(v.x, b) << 24) | (nibble_word_plane_byte(v.y, b) << 16) |
                                  (nibble_word_plane_byte(v.z, b) << 8) | nibble_word_plane_byte(v.w, b);
            planes[(size_t)b * n_words + t] = word;
        }
    }
}

// planes[b][row][KW] -> field-packed K tiles tiled[kt][row][bits * 4 words] (abq_bits.h).
// store_fields puts the field words of word-set `ws` into the record at `rec`.
template <int BITS>
__device__ __forceinline__ void store_fields(uint32_t *rec, int ws, const uint32_t (&f)[BITS])
{
    if constexpr (BITS == 8) {
        uint4 *dst = reinterpret_cast<uint4 *>(rec + 8 * ws);
        dst[0] = make_uint4(f[0], f[1], f[2], f[3]);
        dst[1] = make_uint4(f[4], f[5], f[6], f[7]);
        return;
    }
    if constexpr ((BITS & 4) != 0) {
        constexpr int i = field_list_index(BITS, 4);
        *reinterpret_cast<uint4 *>(rec + field_word_offset(BITS, 4) + 4 * ws) = make_uint4(f[i], f[i + 1], f[i + 2], f[i + 3]);
    }
    if constexpr ((BITS & 2) != 0) {
        constexpr int i = field_list_index(BITS, 2);
        *reinterpret_cast<uint2 *>(rec + field_word_offset(BITS, 2) + 2 * ws) = make_uint2(f[i], f[i + 1]);
    }
    if constexpr ((BITS & 1) != 0)
        rec[field_word_offset(BITS, 1) + ws] = f[field_list_index(BITS, 1)];
}

// Folds a weight zero point into the codes of one word-set: e holds 32 codes, one per byte, as the low `in_bits` bits
// (two's complement when `is_signed`); every code becomes code - z in the low BITS bits.  Returns false where a
// result does not fit BITS bits as a signed number.
template <int BITS> __device__ __forceinline__ bool fold_zero_point(uint32_t (&e)[8], int z, int in_bits, bool is_signed)
{
    bool fits = true;
    const int lo = -(1 << (BITS - 1)), hi = (1 << (BITS - 1)) - 1;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
        uint32_t out = 0;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int code = (int)((e[d] >> (8 * c)) & ((1u << in_bits) - 1u));
            if (is_signed && (code >> (in_bits - 1)))
                code -= 1 << in_bits;
            const int v = code - z;
            fits = fits && v >= lo && v <= hi;
            out |= ((uint32_t)v & ((1u << BITS) - 1u)) << (8 * c);
        }
        e[d] = out;
    }
    return fits;
}

// sums[row] = sum over K of the unsigned codes of a row (bit b of an element counts 2^b): one wave per row, the
// plane words read as 16-byte units along the lanes, a popcount per word and plane.  What the kernels that feed an
// unsigned 8-bit operand as value - 128 add back in their epilogue (GemmArgs::x_row_sums / w_row_sums).
// job: which four rows this workgroup takes.
__device__ __forceinline__ void row_sums_of_four_rows(const uint32_t *__restrict__ planes, int *__restrict__ sums, int rows, int KW,
                                                      int bits, int job)
{
    const int lane = threadIdx.x & 63;
    const int row = job * 4 + (threadIdx.x >> 6);
    if (row >= rows)
        return; // whole waves, no barrier below
    const size_t plane_stride = (size_t)rows * KW;
    unsigned total = 0;
    for (int b = 0; b < bits; ++b) {
        const uint4 *p = reinterpret_cast<const uint4 *>(planes + b * plane_stride + (size_t)row * KW);
        unsigned ones = 0;
        for (int u = lane; u < KW / 4; u += 64) {
            const uint4 v = p[u];
            ones += __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
        }
        total += ones << b;
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1)
        total += __shfl_xor(total, d);
    if (lane == 0)
        sums[row] = (int)total;
}

// One workgroup converts 32 rows x 8 K tiles.  A thread owns one record (one row, one K tile): it
// reads 16 bytes per plane (eight threads cover 128 contiguous bytes of a plane row), converts its
// four word-sets in registers, and parks the record in LDS; the records of one K tile are then
// contiguous in memory over the 32 rows and leave with coalesced 16-byte stores.
// in_bits < BITS: the operand has in_bits planes and is written as records of the wider field (padded records, for
// the widths made of several fields): the planes above it repeat its top plane (sign_extend & 1: signed codes) or
// are zero.  sign_extend & 2 (8-bit records): bit 7 of every code is flipped, i.e. the record holds code - 128
// (biased records of unsigned 8-bit operands, which the signed matrix cores take as they are).
// zero != nullptr (weights with group-wise zero points, group_size a multiple of 32): every code has its group's zero
// point, zero[row][k / group_size], taken off, and the records hold the signed differences; *flag is set where a
// zero point is no whole number or a difference does not fit the records.
template <int BITS>
__global__ __launch_bounds__(256) void relayout_planes_kernel(const uint32_t *__restrict__ planes,
                                                              uint32_t *__restrict__ tiled, int rows, int KW, int in_bits,
                                                              int sign_extend, const float *__restrict__ zero = nullptr,
                                                              int group_size = 0, int *flag = nullptr, int *__restrict__ row_sums = nullptr)
{
    constexpr int REC = BITS * 4;          // words per record
    constexpr int SLAB = 32 * REC + 4;     // words per K tile in LDS (+16 bytes against bank conflicts)
    __shared__ __align__(16) uint32_t buf[8 * SLAB];
    const int tid = threadIdx.x;
    const int kt_tiles = KW / 4;
    // row_sums: the grid has further layers of workgroups behind those that convert, which take the rows' sums of codes
    // from the same planes (one launch instead of two for an operand that needs both)
    if (row_sums && (int)blockIdx.y >= (kt_tiles + 7) / 8) {
        row_sums_of_four_rows(planes, row_sums, rows, KW, in_bits, ((int)blockIdx.y - (kt_tiles + 7) / 8) * (int)gridDim.x + (int)blockIdx.x);
        return;
    }
    const int row0 = blockIdx.x * 32, kt0 = blockIdx.y * 8;
    const size_t plane_stride = (size_t)rows * KW;
    {
        const int i = tid >> 3, j = tid & 7;
        const int row = row0 + i, kt = kt0 + j;
        if (row < rows && kt < kt_tiles) {
            uint32_t pw[4][BITS]; // [word-set][plane]
            const uint32_t *p = planes + (size_t)row * KW + 4 * kt;
#pragma unroll
            for (int b = 0; b < BITS; ++b) {
                uint4 v = *reinterpret_cast<const uint4 *>(p + min(b, in_bits - 1) * plane_stride);
                if (b >= in_bits && !(sign_extend & 1))
                    v = make_uint4(0u, 0u, 0u, 0u);
                pw[0][b] = v.x; pw[1][b] = v.y; pw[2][b] = v.z; pw[3][b] = v.w;
            }
            uint32_t *rec = buf + j * SLAB + i * REC;
#pragma unroll
            for (int ws = 0; ws < 4; ++ws) {
                uint32_t e[8], f[BITS];
                planes_to_int8<BITS, kLow>(pw[ws], e);
                if (BITS == 8 && (sign_extend & 2)) {
#pragma unroll
                    for (int d = 0; d < 8; ++d)
                        e[d] ^= 0x80808080u;
                }
                if (zero) {
                    const float zf = zero[(size_t)row * (KW * 32 / group_size) + (kt * 128 + ws * 32) / group_size];
                    const float zr = rintf(zf);
                    const bool ok = zr == zf && fabsf(zr) <= 256.f && fold_zero_point<BITS>(e, (int)zr, in_bits, (sign_extend & 1) != 0);
                    if (!ok && flag)
                        *flag = 1;
                }
                compress_fields<BITS>(e, f);
                store_fields<BITS>(rec, ws, f);
            }
        }
    }
    __syncthreads();
    const int nrow = min(32, rows - row0);
    for (int j = 0; j < 8; ++j) {
        const int kt = kt0 + j;
        if (kt >= kt_tiles)
            break;
        uint4 *dst = reinterpret_cast<uint4 *>(tiled + ((size_t)kt * rows + row0) * REC);
        const uint4 *src = reinterpret_cast<const uint4 *>(buf + j * SLAB);
        for (int u = tid; u < nrow * BITS; u += 256)
            dst[u] = src[u];
    }
}

// The same with one word-set (32 elements) per thread: a workgroup converts 8 rows x 8 K tiles, 32 consecutive
// threads read 128 contiguous bytes of a plane row.  Four times the workgroups for a quarter of the work each: for
// the few hundred activation rows of a small prefill, where the kernel above would occupy a quarter of the chip
// and its time is one thread's latency chain (512 x 4096 8-bit activations: 64 workgroups there, 256 here).
template <int BITS>
__global__ __launch_bounds__(256) void relayout_planes_ws_kernel(const uint32_t *__restrict__ planes,
                                                                 uint32_t *__restrict__ tiled, int rows, int KW, int in_bits,
                                                                 int sign_extend, int *__restrict__ row_sums = nullptr)
{
    constexpr int REC = BITS * 4;          // words per record
    constexpr int SLAB = 8 * REC + 4;      // words per K tile in LDS (+16 bytes against bank conflicts)
    __shared__ __align__(16) uint32_t buf[8 * SLAB];
    const int tid = threadIdx.x;
    const int kt_tiles = KW / 4;
    if (row_sums && (int)blockIdx.y >= (kt_tiles + 7) / 8) { // (see relayout_planes_kernel)
        row_sums_of_four_rows(planes, row_sums, rows, KW, in_bits, ((int)blockIdx.y - (kt_tiles + 7) / 8) * (int)gridDim.x + (int)blockIdx.x);
        return;
    }
    const int row0 = blockIdx.x * 8, kt0 = blockIdx.y * 8;
    const size_t plane_stride = (size_t)rows * KW;
    {
        const int i = tid >> 5, w = tid & 31; // row, word-set within the 8 K tiles
        const int row = row0 + i, kw = 4 * kt0 + w;
        if (row < rows && kw < KW) {
            uint32_t pw[BITS], e[8], f[BITS];
            const uint32_t *p = planes + (size_t)row * KW + kw;
#pragma unroll
            for (int b = 0; b < BITS; ++b)
                pw[b] = (b >= in_bits && !(sign_extend & 1)) ? 0u : p[min(b, in_bits - 1) * plane_stride];
            planes_to_int8<BITS, kLow>(pw, e);
            if (BITS == 8 && (sign_extend & 2)) {
#pragma unroll
                for (int d = 0; d < 8; ++d)
                    e[d] ^= 0x80808080u;
            }
            compress_fields<BITS>(e, f);
            store_fields<BITS>(buf + (w >> 2) * SLAB + i * REC, w & 3, f);
        }
    }
    __syncthreads();
    const int nrow = min(8, rows - row0);
    const int per_tile = nrow * BITS; // 16-byte units of one K tile's records
    for (int u = tid; u < 8 * per_tile; u += 256) {
        const int j = u / per_tile, v = u - j * per_tile;
        if (kt0 + j < kt_tiles)
            reinterpret_cast<uint4 *>(tiled + ((size_t)(kt0 + j) * rows + row0) * REC)[v] =
                reinterpret_cast<const uint4 *>(buf + j * SLAB)[v];
    }
}

// bits: width of the records written; in_bits <= bits: planes the operand has (sign_extend: what the rest repeats)
// row_sums != nullptr: the rows' sums of codes (as abq_row_sums takes them from the in_bits planes) in the same launch.
hipError_t launch_relayout_planes_padded(const uint32_t *planes, uint32_t *tiled, int rows, int k, int bits, int in_bits,
                                         int sign_extend, hipStream_t stream, int *row_sums)
{
    const int KW = k / 32;
    dim3 grid((rows + 31) / 32, (KW / 4 + 7) / 8);
    const int sum_jobs = row_sums ? (rows + 3) / 4 : 0; // workgroups of four waves, a row each
    if ((long)grid.x * grid.y < 256) { // less than a workgroup per compute unit: the finer kernel
        dim3 fine((rows + 7) / 8, (KW / 4 + 7) / 8);
        fine.y += (sum_jobs + fine.x - 1) / fine.x;
        switch (bits) {
#define ABQ_RELAYOUT_CASE(B)                                                                                     \
    case B:                                                                                                      \
        hipLaunchKernelGGL(relayout_planes_ws_kernel<B>, fine, dim3(256), 0, stream, planes, tiled, rows, KW, in_bits, sign_extend, row_sums); \
        break;
            ABQ_RELAYOUT_CASE(1) ABQ_RELAYOUT_CASE(2) ABQ_RELAYOUT_CASE(3) ABQ_RELAYOUT_CASE(4)
            ABQ_RELAYOUT_CASE(5) ABQ_RELAYOUT_CASE(6) ABQ_RELAYOUT_CASE(7) ABQ_RELAYOUT_CASE(8)
#undef ABQ_RELAYOUT_CASE
        default:
            return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    grid.y += (sum_jobs + grid.x - 1) / grid.x;
    switch (bits) {
#define ABQ_RELAYOUT_CASE(B)                                                                                     \
    case B:                                                                                                      \
        hipLaunchKernelGGL(relayout_planes_kernel<B>, grid, dim3(256), 0, stream, planes, tiled, rows, KW, in_bits, sign_extend, \
                           (const float *)nullptr, 0, (int *)nullptr, row_sums);                                 \
        break;
        ABQ_RELAYOUT_CASE(1) ABQ_RELAYOUT_CASE(2) ABQ_RELAYOUT_CASE(3) ABQ_RELAYOUT_CASE(4)
        ABQ_RELAYOUT_CASE(5) ABQ_RELAYOUT_CASE(6) ABQ_RELAYOUT_CASE(7) ABQ_RELAYOUT_CASE(8)
#undef ABQ_RELAYOUT_CASE
    default:
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Records of `bits` bits holding code - zero point (see relayout_planes_kernel).
hipError_t launch_relayout_planes_folded(const uint32_t *planes, const float *zero, int group_size, uint32_t *tiled, int rows, int k,
                                         int bits, int in_bits, int is_signed, int *flag, hipStream_t stream)
{
    const int KW = k / 32;
    const dim3 grid((rows + 31) / 32, (KW / 4 + 7) / 8);
    switch (bits) {
#define ABQ_RELAYOUT_CASE(B)                                                                                     \
    case B:                                                                                                      \
        hipLaunchKernelGGL(relayout_planes_kernel<B>, grid, dim3(256), 0, stream, planes, tiled, rows, KW, in_bits, is_signed ? 1 : 0, \
                           zero, group_size, flag);                                                              \
        break;
        ABQ_RELAYOUT_CASE(2) ABQ_RELAYOUT_CASE(4) ABQ_RELAYOUT_CASE(8)
#undef ABQ_RELAYOUT_CASE
    default:
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_relayout_planes(const uint32_t *planes, uint32_t *tiled, int rows, int k, int bits, hipStream_t stream)
{
    return launch_relayout_planes_padded(planes, tiled, rows, k, bits, bits, 0, stream, nullptr);
}

// ---- FP6 records ---------------------------------------------------------------------------
//
// Operand format of the FP6 MFMA kernel (abq_gemm_fp6.hip).  An element becomes the 6-bit
// sign-magnitude code (sign << 5) | |value|, which read as an E2M3 float is value / 8 for every
// |value| <= 16.  A word-set (32 consecutive K elements, one plane word) becomes a string of
// 192 bits: position p (bits [6p, 6p+6)) holds element 31 - 8 (p % 4) - p / 4, the order the
// bit-matrix transpose leaves them in; both operands use it, and a dot product does not care.
// A row's K tile of 128 elements is one record of 24 words, word-set ws at words
// [12 (ws & 1) + 6 (ws >> 1), +6): the two word-sets that lanes 0-31 feed to the two MFMA
// K steps come first, then the two of lanes 32-63.  Records are stored fp6[kt][row][24].

// r[0..4]: bit-sliced magnitude, r[5]: sign, r[6], r[7]: zero -> the word-set's string of 6-bit codes.
__device__ __forceinline__ void fp6_string_of_codes(uint32_t (&r)[8], uint32_t (&out)[6])
{
    transpose8x8x4(r); // dword d, byte c: the code of the element at plane bit 8c + d
    uint32_t y[8];
#pragma unroll
    for (int d = 0; d < 8; ++d)
        y[d] = (r[d] & 0x3Fu) | ((r[d] >> 2) & 0xFC0u) | ((r[d] >> 4) & 0x3F000u) | ((r[d] >> 6) & 0xFC0000u);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        out[3 * h + 0] = y[4 * h] | (y[4 * h + 1] << 24);
        out[3 * h + 1] = (y[4 * h + 1] >> 8) | (y[4 * h + 2] << 16);
        out[3 * h + 2] = (y[4 * h + 2] >> 16) | (y[4 * h + 3] << 8);
    }
}

// Bit-sliced |value| and sign of 32 elements: p[t] = plane t, planes at and above bits - 1 read
// as the sign plane (two's complement sign extension) when the operand is signed.
__device__ __forceinline__ void fp6_string(const uint32_t (&p)[5], int bits, bool is_signed, uint32_t (&out)[6])
{
    const uint32_t s = is_signed ? p[bits - 1] : 0u;
    uint32_t r[8];
    uint32_t carry = s; // |v| = (v ^ -sign) + sign, one ripple step per plane
#pragma unroll
    for (int t = 0; t < 5; ++t) {
        const uint32_t x = ((t < bits - 1 || !is_signed) && t < bits ? p[t] : s) ^ s;
        r[t] = x ^ carry;
        carry &= x;
    }
    r[5] = s;
    r[6] = 0u;
    r[7] = 0u;
    fp6_string_of_codes(r, out);
}

// The same for code - z (a weight zero point folded in): the difference of the bit-sliced codes and the constant as six
// planes of two's complement, then sign and magnitude as above.  Returns a word with a bit set for every element whose
// difference has a magnitude above 16 (no E2M3 number).  |z| <= 32.
__device__ __forceinline__ uint32_t fp6_string_folded(const uint32_t (&p)[5], int bits, bool is_signed, int z, uint32_t (&out)[6])
{
    uint32_t d[6], borrow = 0u;
#pragma unroll
    for (int t = 0; t < 6; ++t) {
        const uint32_t a = t < bits ? p[t] : (is_signed ? p[bits - 1] : 0u);
        const uint32_t zb = ((z >> t) & 1) ? 0xFFFFFFFFu : 0u;
        d[t] = a ^ zb ^ borrow;
        borrow = (~a & zb) | (~(a ^ zb) & borrow);
    }
    const uint32_t s = d[5];
    uint32_t r[8], carry = s;
#pragma unroll
    for (int t = 0; t < 5; ++t) {
        const uint32_t x = d[t] ^ s;
        r[t] = x ^ carry;
        carry &= x;
    }
    const uint32_t misfit = carry | (r[4] & (r[0] | r[1] | r[2] | r[3])); // -32, or a magnitude of 17 .. 31
    r[5] = s;
    r[6] = 0u;
    r[7] = 0u;
    fp6_string_of_codes(r, out);
    return misfit;
}


// One thread per word-set; a workgroup covers 8 rows x 8 K tiles (32 consecutive plane words of a
// row are one coalesced 128-byte read per plane) and writes each tile's 8 records (contiguous in
// memory) with 16-byte stores out of LDS.
// zero != nullptr (weights with group-wise zero points, group_size a multiple of 32): the records hold code - zero
// point, zero[row][k / group_size]; *flag is set where a zero point is no whole number or a difference has no FP6 code.
template <int BITS>
__global__ __launch_bounds__(256) void relayout_planes_fp6_kernel(const uint32_t *__restrict__ planes,
                                                                  uint32_t *__restrict__ fp6, int rows, int KW,
                                                                  int is_signed, const float *__restrict__ zero = nullptr,
                                                                  int group_size = 0, int *flag = nullptr)
{
    constexpr int REC = 24;
    constexpr int SLAB = 8 * REC + 4; // words per K tile in LDS (+16 bytes against bank conflicts)
    __shared__ __align__(16) uint32_t buf[8 * SLAB];
    const int tid = threadIdx.x;
    const int kt_tiles = KW / 4;
    const int row0 = blockIdx.x * 8, kt0 = blockIdx.y * 8;
    const size_t plane_stride = (size_t)rows * KW;
    {
        const int i = tid >> 5, w = tid & 31; // row, word-set within the 8 tiles
        const int row = row0 + i, kw = 4 * kt0 + w;
        if (row < rows && kw < KW) {
            uint32_t pw[5];
            const uint32_t *p = planes + (size_t)row * KW + kw;
#pragma unroll
            for (int b = 0; b < 5; ++b)
                pw[b] = b < BITS ? p[b * plane_stride] : 0u;
            uint32_t o[6];
            if (zero) {
                const float zf = zero[(size_t)row * (KW * 32 / group_size) + kw * 32 / group_size];
                const float zr = rintf(zf);
                const bool whole = zr == zf && fabsf(zr) <= 31.f;
                const uint32_t misfit = fp6_string_folded(pw, BITS, is_signed != 0, whole ? (int)zr : 0, o);
                if ((!whole || misfit) && flag)
                    *flag = 1;
            } else {
                fp6_string(pw, BITS, is_signed != 0, o);
            }
            const int ws = w & 3;
            uint32_t *rec = buf + (w >> 2) * SLAB + i * REC + 12 * (ws & 1) + 6 * (ws >> 1);
            *reinterpret_cast<uint2 *>(rec) = make_uint2(o[0], o[1]);
            *reinterpret_cast<uint2 *>(rec + 2) = make_uint2(o[2], o[3]);
            *reinterpret_cast<uint2 *>(rec + 4) = make_uint2(o[4], o[5]);
        }
    }
    __syncthreads();
    const int nrow = min(8, rows - row0);
    const int per_tile = nrow * (REC / 4); // 16-byte pieces per K tile
    for (int u = tid; u < 8 * per_tile; u += 256) {
        const int j = u / per_tile, q = u % per_tile;
        const int kt = kt0 + j;
        if (kt < kt_tiles)
            reinterpret_cast<uint4 *>(fp6 + ((size_t)kt * rows + row0) * REC)[q] =
                reinterpret_cast<const uint4 *>(buf + j * SLAB)[q];
    }
}

__global__ __launch_bounds__(256) void row_sums_kernel(const uint32_t *__restrict__ planes, int *__restrict__ sums, int rows,
                                                       int KW, int bits)
{
    row_sums_of_four_rows(planes, sums, rows, KW, bits, blockIdx.x);
}

hipError_t launch_row_sums(const uint32_t *planes, int *sums, int rows, int k, int bits, hipStream_t stream)
{
    hipLaunchKernelGGL(row_sums_kernel, dim3((rows + 3) / 4), dim3(256), 0, stream, planes, sums, rows, k / 32, bits);
    return hipGetLastError();
}

hipError_t launch_relayout_planes_fp6(const uint32_t *planes, uint32_t *fp6, int rows, int k, int bits, int is_signed,
                                      hipStream_t stream, const float *zero, int group_size, int *flag)
{
    const int KW = k / 32;
    const dim3 grid((rows + 7) / 8, (KW / 4 + 7) / 8);
    switch (bits) {
#define ABQ_FP6_CASE(B)                                                                                                  \
    case B:                                                                                                              \
        hipLaunchKernelGGL(relayout_planes_fp6_kernel<B>, grid, dim3(256), 0, stream, planes, fp6, rows, KW, is_signed, zero, \
                           group_size, flag);                                                                            \
        break;
        ABQ_FP6_CASE(1) ABQ_FP6_CASE(2) ABQ_FP6_CASE(3) ABQ_FP6_CASE(4) ABQ_FP6_CASE(5)
#undef ABQ_FP6_CASE
    default:
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// compress_fields + store_fields for a run-time bit width
template <int BITS> __device__ __forceinline__ void store_fields_of(uint32_t *rec, int ws, const uint32_t (&e)[8])
{
    uint32_t f[BITS];
    compress_fields<BITS>(e, f);
    store_fields<BITS>(rec, ws, f);
}

__device__ __forceinline__ void store_fields_any(uint32_t *rec, int ws, const uint32_t (&e)[8], int bits)
{
    switch (bits) {
    case 1: store_fields_of<1>(rec, ws, e); break;
    case 2: store_fields_of<2>(rec, ws, e); break;
    case 3: store_fields_of<3>(rec, ws, e); break;
    case 4: store_fields_of<4>(rec, ws, e); break;
    case 5: store_fields_of<5>(rec, ws, e); break;
    case 6: store_fields_of<6>(rec, ws, e); break;
    case 7: store_fields_of<7>(rec, ws, e); break;
    default: store_fields_of<8>(rec, ws, e); break;
    }
}

// ---- per-token dynamic quantisation fused with packing ------------------------------------
//
// One workgroup per token row of fp16 activations [M][K]: min / max of the row, scale and zero
// point as the reference's per_token_dynamic_calibration derives them
// (algorithm/quantize/quantizer.py:149-179), integer codes as its fake_quant rounds and clamps
// them (:120-123), then the bit planes of the codes.  Codes leave as signed two's complement:
//   symmetric : scale = clamp(absmax / (2^(n-1)-1), 1e-5, 1e4), code = clamp(rint(x/scale), -2^(n-1), 2^(n-1)-1)
//   asymmetric: scale = clamp((max-min) / (2^n-1), 1e-5, 1e4), zp = rint(clamp(-min/scale, -1e4, 1e4)),
//               u = clamp(rint(x/scale) + zp, 0, 2^n-1); stored code = u - 2^(n-1), zero = zp - 2^(n-1)
// so that x ~ scale * (code - zero) either way (zero = 0 when symmetric).  Arithmetic is fp32.
// Optionally writes the sum of the codes over every group of group_size elements (the GEMM's
// zero-point correction needs them).

// Writes the word-set w (32 elements) of `row` into the field-packed K-tiled records tiled[kt][row][bits * 4];
// the quad's lane q holds the elements 8q..8q+7 of the word-set, of which the low `bits` bits are kept.
__device__ __forceinline__ void emit_tiled(const int (&v)[8], uint32_t *tiled, int rows, int row, int w, int quad_lane,
                                           int bits, bool active, uint32_t sel_pair, uint32_t sel_half)
{
    if (bits == 8) {
        // 8-bit codes are the record's bytes themselves: expanded dword s, byte c = element 31 - (8c + s) of
        // the word-set = element 7 - s of lane 3 - c.  The quad transposes its bytes so that lane s ends
        // with the dwords 2 s and 2 s + 1, which it stores as one piece of 8 bytes: sixteen lanes cover a
        // record's 128 bytes with one store instruction.
        const uint32_t e_even = quad_transpose_bytes(pack_low_bytes(v[7], v[5], v[3], v[1]), sel_pair, sel_half);
        const uint32_t e_odd = quad_transpose_bytes(pack_low_bytes(v[6], v[4], v[2], v[0]), sel_pair, sel_half);
        if (active) {
            uint32_t *dst = tiled + ((size_t)(w >> 2) * rows + row) * 32 + 8 * (w & 3) + 2 * quad_lane;
            *reinterpret_cast<uint2 *>(dst) = make_uint2(e_even, e_odd);
        }
        return;
    }
    // expanded dword s, byte c = element 31 - (8c + s) of the word-set: this lane's element
    // 7 - s goes to byte 3 - quad_lane
    const uint32_t pattern_mask = (1u << bits) - 1u;
    uint32_t e[8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
        e[s] = quad_or(((uint32_t)v[7 - s] & pattern_mask) << (24 - 8 * quad_lane));
    if (active && quad_lane == 0)
        store_fields_any(tiled + ((size_t)(w >> 2) * rows + row) * (bits * 4), w & 3, e, bits);
}

// Eight codes of magnitude at most 16 (this lane's unit: elements 8 u .. 8 u + 7 of `row`, u = 4 w + quad_lane) ->
// their share of the row's FP6 record; the four lanes of a quad assemble one word-set of 192 bits.
__device__ __forceinline__ void emit_fp6(const int (&v)[8], uint32_t *records, int rows, int row, int w, int quad_lane, bool active)
{
    // position p = 4 s + c of the word-set's 192-bit string holds element 31 - (8c + s): this lane's
    // element j goes to position 4 (7 - j) + 3 - quad_lane as the code (sign << 5) | magnitude
    uint32_t o[6] = { 0u, 0u, 0u, 0u, 0u, 0u };
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t code = v[j] < 0 ? (32u | (uint32_t)(-v[j])) : (uint32_t)v[j];
        constexpr int kBase[8] = { 168, 144, 120, 96, 72, 48, 24, 0 }; // 24 (7 - j)
        const int d0 = kBase[j] >> 5;                                   // first dword the code can touch
        const uint64_t wide = (uint64_t)code << ((kBase[j] & 31) + 6 * (3 - quad_lane));
        o[d0] |= (uint32_t)wide;
        if (d0 + 1 < 6)
            o[d0 + 1] |= (uint32_t)(wide >> 32);
    }
#pragma unroll
    for (int d = 0; d < 6; ++d)
        o[d] = quad_or(o[d]);
    if (active && quad_lane == 0) {
        const int ws = w & 3;
        uint32_t *rec = records + ((size_t)(w >> 2) * rows + row) * 24 + 12 * (ws & 1) + 6 * (ws >> 1);
        *reinterpret_cast<uint2 *>(rec) = make_uint2(o[0], o[1]);
        *reinterpret_cast<uint2 *>(rec + 2) = make_uint2(o[2], o[3]);
        *reinterpret_cast<uint2 *>(rec + 4) = make_uint2(o[4], o[5]);
    }
}

// pack_f16_kernel's values (fp16 product with the scale, truncated, no clamp: abq_gemm_wrapper.cu:29-54 of the
// reference), written as field-packed K-tiled records instead of planes: what relayout_planes_kernel makes of
// pack_f16_kernel's output, in one pass.
// FP6: the same values written as FP6 records (codes of at most 5 bits signed / 4 unsigned): the low `bits` bits of
// the truncated product, read as the signed or unsigned code they are in the planes (values beyond the range alias
// there as well: the reference packs the low bits and does not clamp).
template <bool FP6>
__global__ __launch_bounds__(256) void pack_f16_tiled_kernel(const uint4 *__restrict__ in, const float *__restrict__ scale,
                                                             uint32_t *__restrict__ tiled, int rows, int units, int bits,
                                                             int is_signed)
{
    const _Float16 hs = (_Float16)scale[0];
    const size_t n_units = (size_t)rows * units; // units per row: a multiple of 16, so a quad is active as one
    const size_t rounded = (n_units + 255) / 256 * 256;
    uint32_t sel_pair, sel_half;
    quad_transpose_selectors(threadIdx.x & 3, sel_pair, sel_half);
    for (size_t t = (size_t)blockIdx.x * 256 + threadIdx.x; t < rounded; t += (size_t)gridDim.x * 256) {
        const bool active = t < n_units;
        int v[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
        if (active) {
            union {
                uint4 u;
                _Float16 h[8];
            } raw;
            raw.u = in[t];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const _Float16 p = raw.h[c] * hs; // fp16 product, rounded to nearest even
                v[c] = (int)p;                    // truncation
            }
        }
        const int row = (int)(t / units), u = (int)(t % units);
        if constexpr (FP6) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const int low = v[c] & ((1 << bits) - 1);
                v[c] = (is_signed && (low >> (bits - 1))) ? low - (1 << bits) : low;
            }
            emit_fp6(v, tiled, rows, active ? row : 0, u >> 2, u & 3, active);
        } else {
            emit_tiled(v, tiled, rows, active ? row : 0, u >> 2, u & 3, bits, active, sel_pair, sel_half);
        }
    }
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// Quantises the eight fp16 values of unit u (elements 8u .. 8u + 7) of `row` and writes their share of the
// packed row; the lanes of a quad hold consecutive units (quad_lane = u & 3), a scale group's lanes are
// consecutive too.  Inactive lanes (units past the row) take part in the cross-lane steps with zeros.
// BITS: the code width where the instantiation fixes it (8), 0 where it is the run-time argument.
template <int LAYOUT, int BITS = 0>
__device__ __forceinline__ void quant_emit_unit(const uint4 &rawq, bool active, int u, int row, int M, int K, int bits_arg,
                                                const QuantRow &q, uint32_t *planes, int *group_sums, int group_size,
                                                uint32_t sel_pair, uint32_t sel_half)
{
    const int bits = BITS ? BITS : bits_arg;
    const int KW = K / 32;
    const int lanes_per_group = group_size / 8;
    int v[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
    int sum = 0;
    if (active) {
        union {
            uint4 q;
            _Float16 h[8];
        } raw;
        raw.q = rawq;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            v[c] = quant_code((float)raw.h[c], q);
            sum += v[c];
        }
    }
    if (group_sums) {
        const int glog = group_size == 64 ? 3 : 4; // lanes of a scale group: 8 or 16
        for (int o = 1; o < lanes_per_group; o <<= 1)
            sum += __shfl_xor(sum, o);
        if (active && (u & (lanes_per_group - 1)) == 0)
            group_sums[(size_t)row * (K >> (glog + 3)) + (u >> glog)] = sum;
    }
    const int quad_lane = u & 3, w = u >> 2; // w: word-set (32 elements) within the row
    if (LAYOUT == 2) {
        emit_fp6(v, planes, M, row, w, quad_lane, active);
    } else if (LAYOUT == 1) {
        emit_tiled(v, planes, M, row, w, quad_lane, bits, active, sel_pair, sel_half);
    } else {
        const uint64_t bytes = eight_values_to_plane_bytes(v);
        for (int b = 0; b < bits; ++b) {
            uint32_t word = (uint32_t)((bytes >> (8 * b)) & 0xFFu) << (24 - 8 * quad_lane);
            word = quad_or(word);
            if (active && quad_lane == 0)
                planes[((size_t)b * M + row) * KW + w] = word;
        }
    }
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// One WAVE per token row, the row held in registers between the two passes: NU 16-byte units per lane are all in
// flight at once, there is no barrier and no LDS round trip, and the waves of a compute unit are each at their
// own point of their rows, so loads, arithmetic and stores of different rows overlap.  (With one workgroup per
// row, a row's loads were in flight only during the first third of the workgroup's life: 3.2 TB/s where a plain
// copy of the same buffers reaches 5.5.)  Rows of up to NU * 512 elements, NU <= 24 (beyond, the row spills).
// WPR = 4: the four waves of a workgroup share one row (wave w takes the rounds of 64 units w, w + 4, ...; NU is then
// what one wave holds) and exchange their extrema through LDS: for the few hundred to two thousand rows of a small
// prefill, where one wave per row leaves a SIMD with one or two waves and the time is a wave's own chain of
// instructions (914 at K = 4096, 2359 at K = 11008) behind the latency of its loads.
template <int LAYOUT, int NU, int BITS, int WPR = 1>
__global__ __launch_bounds__(256) void quant_pack_wave_rows_kernel(const uint4 *__restrict__ x, uint32_t *__restrict__ planes,
                                                                   float *__restrict__ scale_out, float *__restrict__ zero_out,
                                                                   int *__restrict__ group_sums, int M, int K, int bits,
                                                                   int symmetric, int group_size)
{
    static_assert(WPR == 1 || WPR == 4, "one wave or the whole workgroup per row");
    const int lane = threadIdx.x & 63;
    const int wsub = WPR == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // the wave's place in its row
    const int row = WPR == 1 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
    if (row >= M)
        return; // whole waves leave: nothing below synchronises across waves (WPR = 4: the grid has M workgroups)
    const int units = K / 8;
    const uint4 *xr = x + (size_t)row * units;
    uint4 raw[NU];
#pragma unroll
    for (int i = 0; i < NU; ++i) {
        const int u = lane + 64 * (i * WPR + wsub);
        // (read once: non-temporal; past the end: the row's first unit once more, it changes no extremum)
        typedef unsigned int unit_words __attribute__((ext_vector_type(4)));
        const unit_words w = __builtin_nontemporal_load(reinterpret_cast<const unit_words *>(xr + (u < units ? u : 0)));
        raw[i] = make_uint4(w.x, w.y, w.z, w.w);
    }
    half2_t mx2 = { (_Float16)-INFINITY, (_Float16)-INFINITY }, mn2 = { (_Float16)INFINITY, (_Float16)INFINITY };
#pragma unroll
    for (int i = 0; i < NU; ++i) {
        union {
            uint4 q;
            half2_t h2[4];
        } r;
        r.q = raw[i];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            mx2 = __builtin_elementwise_max(mx2, r.h2[c]);
            mn2 = __builtin_elementwise_min(mn2, r.h2[c]);
        }
    }
    float mx = fmaxf((float)mx2.x, (float)mx2.y), mn = fminf((float)mn2.x, (float)mn2.y);
    mx = wave_max(mx);
    mn = -wave_max(-mn);
    if constexpr (WPR > 1) {
        __shared__ float red[2][WPR];
        if (lane == 0) {
            red[0][wsub] = mx;
            red[1][wsub] = mn;
        }
        __syncthreads();
#pragma unroll
        for (int w = 0; w < WPR; ++w) {
            mx = fmaxf(mx, red[0][w]);
            mn = fminf(mn, red[1][w]);
        }
    }
    const QuantRow q = quant_row_params(mx, mn, bits, symmetric);
    if (lane == 0 && wsub == 0) {
        scale_out[row] = q.scale;
        if (zero_out)
            zero_out[row] = q.zero_out;
    }
    uint32_t sel_pair, sel_half;
    quad_transpose_selectors(lane & 3, sel_pair, sel_half);
    // a row that holds an infinity (or a NaN) takes the general path, whose quotients get the division's fix-up
    const bool finite_row = __builtin_amdgcn_readfirstlane(fabsf(mx) <= 65504.f && fabsf(mn) <= 65504.f) != 0;
    if (LAYOUT == 1 && BITS == 8 && finite_row) {
        // The common case written out: 8-bit codes into K-tiled records.  Per unit: eight quotients, two byte
        // packs, the group sum as two dot products with ones and a butterfly of row operations over the
        // group's 8 or 16 lanes, two 4 x 4 byte transposes across the quad, one 8-byte store.  Unit
        // u = lane + 64 j (round j = i, or i * WPR + the wave's place) lies in K tile (lane >> 4) + 4 j: a fixed stride
        // between a lane's records.
        // clamp(rint(q) + zp, lo, hi) = rint(clamp(q, lo - zp, hi - zp)) + zp (the bounds are integers), and
        // adding 1.5 * 2^23 to a float of magnitude below 2^22 rounds it to an integer, to nearest even like rint,
        // and leaves that integer in the low mantissa bits: clamp, add, integer subtract.
        const float q_lo = q.lo_stored - q.zp_stored, q_hi = q.hi_stored - q.zp_stored;
        const float magic = 12582912.0f; // 1.5 * 2^23
        const int unmagic = 0x4B400000 - (int)q.zp_stored;
        uint32_t *rec = planes + ((size_t)(lane >> 4) * M + row) * 32 + 8 * ((lane >> 2) & 3) + 2 * (lane & 3);
        const size_t rec_stride = (size_t)4 * M * 32;
        const int glog = group_size == 64 ? 3 : 4; // lanes of a scale group
        int *gs = group_sums ? group_sums + (size_t)row * (K / group_size) + (lane >> glog) : nullptr;
        const int gs_stride = 64 >> glog;
        const bool gs_lane = (lane & ((1 << glog) - 1)) == 0;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const int j = i * WPR + wsub; // the round of 64 units
            if (64 * (j + 1) <= units) { // wave-uniform: every lane has a unit
                union {
                    uint4 q;
                    _Float16 h[8];
                } r;
                r.q = raw[i];
                int v[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const float xf = (float)r.h[c];
                    const float t = xf * q.recip;
                    const float quotient = __builtin_fmaf(__builtin_fmaf(-t, q.scale, xf), q.recip, t);
                    v[c] = __builtin_bit_cast(int, __builtin_amdgcn_fmed3f(quotient, q_lo, q_hi) + magic) - unmagic;
                }
                const uint32_t pa = pack_low_bytes(v[7], v[5], v[3], v[1]), pb = pack_low_bytes(v[6], v[4], v[2], v[0]);
                if (gs) {
                    int sum = __builtin_amdgcn_sdot4((int)pa, 0x01010101, __builtin_amdgcn_sdot4((int)pb, 0x01010101, 0, false), false);
                    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
                    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
                    sum += __builtin_amdgcn_update_dpp(0, sum, 0x141, 0xF, 0xF, true); // row_half_mirror
                    if (glog == 4)
                        sum += __builtin_amdgcn_update_dpp(0, sum, 0x140, 0xF, 0xF, true); // row_mirror
                    if (gs_lane)
                        gs[j * gs_stride] = sum;
                }
                const uint32_t e_even = quad_transpose_bytes(pa, sel_pair, sel_half);
                const uint32_t e_odd = quad_transpose_bytes(pb, sel_pair, sel_half);
                *reinterpret_cast<uint2 *>(rec + j * rec_stride) = make_uint2(e_even, e_odd);
            } else if (64 * j < units) { // the row's last, partly filled round
                const int u = lane + 64 * j;
                quant_emit_unit<LAYOUT, BITS>(raw[i], u < units, u, row, M, K, bits, q, planes, group_sums, group_size, sel_pair, sel_half);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const int j = i * WPR + wsub, u = lane + 64 * j;
            if (64 * j < units) // wave-uniform: units is a multiple of 16, so quads and groups are active as one
                quant_emit_unit<LAYOUT, BITS>(raw[i], u < units, u, row, M, K, bits, q, planes, group_sums, group_size, sel_pair, sel_half);
        }
    }
}

// LAYOUT: 0 planes, 1 field-packed K tiles, 2 FP6 records (codes of at most 5 bits).
template <int LAYOUT>
__global__ __launch_bounds__(256) void quant_pack_rows_kernel(const uint4 *__restrict__ x, uint32_t *__restrict__ planes,
                                                              float *__restrict__ scale_out, float *__restrict__ zero_out,
                                                              int *__restrict__ group_sums, int M, int K, int bits,
                                                              int symmetric, int group_size, int keep_row)
{
    // keep_row: the row stays in LDS between the two passes (each lane re-reads the units it wrote itself),
    // so that it comes from memory once; with rows of 22 KB the rows in flight no longer fit the L2
    extern __shared__ uint4 row_lds[];
    __shared__ float red[2][4];
    const int row = blockIdx.x, tid = threadIdx.x;
    const int units = K / 8; // 8 halves per 16-byte load
    const uint4 *xr = x + (size_t)row * units;

    // four loads in flight per lane: with one, the pass is bound by the latency of memory, not its bandwidth.
    // Minimum and maximum are taken on the fp16 pairs as they are (two elements per instruction).
    half2_t mx2 = { (_Float16)-INFINITY, (_Float16)-INFINITY }, mn2 = { (_Float16)INFINITY, (_Float16)INFINITY };
    for (int u0 = tid; u0 < units; u0 += 1024) {
        union {
            uint4 q;
            half2_t h2[4];
        } raw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int u = u0 + 256 * i;
            raw[i].q = xr[u < units ? u : u0]; // past the end: the lane's first unit once more
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int u = u0 + 256 * i;
            if (keep_row && u < units)
                row_lds[u] = raw[i].q;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                mx2 = __builtin_elementwise_max(mx2, raw[i].h2[c]);
                mn2 = __builtin_elementwise_min(mn2, raw[i].h2[c]);
            }
        }
    }
    float mx = fmaxf((float)mx2.x, (float)mx2.y), mn = fminf((float)mn2.x, (float)mn2.y);
    mx = wave_max(mx);
    mn = -wave_max(-mn);
    if ((tid & 63) == 0) {
        red[0][tid >> 6] = mx;
        red[1][tid >> 6] = mn;
    }
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    mn = fminf(fminf(red[1][0], red[1][1]), fminf(red[1][2], red[1][3]));

    const QuantRow q = quant_row_params(mx, mn, bits, symmetric);
    if (tid == 0) {
        scale_out[row] = q.scale;
        if (zero_out)
            zero_out[row] = q.zero_out;
    }
    const int rounded = (units + 255) / 256 * 256;
    uint32_t sel_pair, sel_half;
    quad_transpose_selectors(tid & 3, sel_pair, sel_half);
    for (int u = tid; u < rounded; u += 256) {
        const bool active = u < units; // units is a multiple of 16: quads and groups are active as one
        uint4 rawq = make_uint4(0u, 0u, 0u, 0u);
        if (active)
            rawq = keep_row ? row_lds[u] : xr[u];
        quant_emit_unit<LAYOUT>(rawq, active, u, row, M, K, bits, q, planes, group_sums, group_size, sel_pair, sel_half);
    }
}

hipError_t launch_quant_pack_rows(const void *x, uint32_t *planes, float *scale, float *zero, int *group_sums,
                                  int M, int K, int bits, int symmetric, int group_size, int layout,
                                  hipStream_t stream)
{
    const int nu = (K + 511) / 512; // rounds of 64 units (512 elements) in a row
    // A workgroup per row, a quarter of the row's rounds per wave, while one wave per row would leave the SIMDs with a
    // wave or two each; the longer the row, the more rows that is (a lone wave holding 16 to 24 units per lane runs at a
    // lower occupancy as well).  8-bit codes into K-tiled records with group sums, one wave per row -> four, us:
    // K = 4096: 64 rows 5.3 -> 3.6, 512 5.6 -> 4.4, 1024 6.1 -> 5.5, 2048 8.3 -> 8.6; K = 2048: 256 4.1 -> 3.3, 2048 5.4 -> 6.2;
    // K = 5120: 1024 7.4 -> 6.4, 4096 16.9 -> 17.4; K = 8192: 4096 26.2 -> 24.1, 16384 75.9 -> 83.6; K = 11008: 1024
    // 13.4 -> 10.3, 8192 60.1 -> 54.2, 16384 107.8 -> 113.5; K = 13824 (against the kernel that keeps the row in LDS):
    // 1024 16.4 -> 11.9, 16384 177 -> 142.
    const int split_rows = nu <= 2 ? 256 : nu <= 8 ? 1024 : nu <= 12 ? 2048 : nu <= 16 ? 4096 : nu <= 24 ? 8192 : INT_MAX;
    if (nu <= 32 && M <= split_rows) {
        const dim3 grid(M), block(256);
        const int nu4 = (nu + 3) / 4;
#define ABQ_QP_SPLIT(L, NU)                                                                                                 \
    do {                                                                                                                    \
        if (L == 1 && bits == 8)                                                                                            \
            hipLaunchKernelGGL((quant_pack_wave_rows_kernel<L, NU, (L == 1 ? 8 : 0), 4>), grid, block, 0, stream,              \
                               reinterpret_cast<const uint4 *>(x), planes, scale, zero, group_sums, M, K, bits, symmetric,  \
                               group_size);                                                                                 \
        else                                                                                                                \
            hipLaunchKernelGGL((quant_pack_wave_rows_kernel<L, NU, 0, 4>), grid, block, 0, stream,                            \
                               reinterpret_cast<const uint4 *>(x), planes, scale, zero, group_sums, M, K, bits, symmetric,  \
                               group_size);                                                                                 \
    } while (0)
#define ABQ_QP_SPLIT_NU(L)       \
    do {                         \
        if (nu4 <= 1)            \
            ABQ_QP_SPLIT(L, 1);  \
        else if (nu4 <= 2)       \
            ABQ_QP_SPLIT(L, 2);  \
        else if (nu4 <= 4)       \
            ABQ_QP_SPLIT(L, 4);  \
        else if (nu4 <= 6)       \
            ABQ_QP_SPLIT(L, 6);  \
        else                     \
            ABQ_QP_SPLIT(L, 8);  \
    } while (0)
        if (layout == 2)
            ABQ_QP_SPLIT_NU(2);
        else if (layout == 1)
            ABQ_QP_SPLIT_NU(1);
        else
            ABQ_QP_SPLIT_NU(0);
#undef ABQ_QP_SPLIT_NU
#undef ABQ_QP_SPLIT
        return hipGetLastError();
    }
    // More rows than that: one wave per row, the row in registers (up to 12288 elements).
    if (nu <= 24) {
        const dim3 grid((M + 3) / 4), block(256);
#define ABQ_QP_WAVE(L, NU)                                                                                                  \
    do {                                                                                                                    \
        if (L == 1 && bits == 8)                                                                                            \
            hipLaunchKernelGGL((quant_pack_wave_rows_kernel<L, NU, (L == 1 ? 8 : 0)>), grid, block, 0, stream,                 \
                               reinterpret_cast<const uint4 *>(x), planes, scale, zero, group_sums, M, K, bits, symmetric,  \
                               group_size);                                                                                 \
        else                                                                                                                \
            hipLaunchKernelGGL((quant_pack_wave_rows_kernel<L, NU, 0>), grid, block, 0, stream,                               \
                               reinterpret_cast<const uint4 *>(x), planes, scale, zero, group_sums, M, K, bits, symmetric,  \
                               group_size);                                                                                 \
    } while (0)
#define ABQ_QP_WAVE_NU(L)       \
    do {                        \
        if (nu <= 2)            \
            ABQ_QP_WAVE(L, 2);  \
        else if (nu <= 4)       \
            ABQ_QP_WAVE(L, 4);  \
        else if (nu <= 8)       \
            ABQ_QP_WAVE(L, 8);  \
        else if (nu <= 16)      \
            ABQ_QP_WAVE(L, 16); \
        else                    \
            ABQ_QP_WAVE(L, 24); \
    } while (0)
        if (layout == 2)
            ABQ_QP_WAVE_NU(2);
        else if (layout == 1)
            ABQ_QP_WAVE_NU(1);
        else
            ABQ_QP_WAVE_NU(0);
#undef ABQ_QP_WAVE_NU
#undef ABQ_QP_WAVE
        return hipGetLastError();
    }
    // a row of up to 48 KiB is kept in LDS (within the default limit together with the static part)
    const int keep_row = (size_t)K * 2 <= 48 * 1024;
    const size_t lds = keep_row ? (size_t)K * 2 : 0;
    if (layout == 2)
        hipLaunchKernelGGL(quant_pack_rows_kernel<2>, dim3(M), dim3(256), lds, stream,
                           reinterpret_cast<const uint4 *>(x), planes, scale, zero, group_sums, M, K, bits,
                           symmetric, group_size, keep_row);
    else if (layout == 1)
        hipLaunchKernelGGL(quant_pack_rows_kernel<1>, dim3(M), dim3(256), lds, stream,
                           reinterpret_cast<const uint4 *>(x), planes, scale, zero, group_sums, M, K, bits,
                           symmetric, group_size, keep_row);
    else
        hipLaunchKernelGGL(quant_pack_rows_kernel<0>, dim3(M), dim3(256), lds, stream,
                           reinterpret_cast<const uint4 *>(x), planes, scale, zero, group_sums, M, K, bits,
                           symmetric, group_size, keep_row);
    return hipGetLastError();
}

// w_zero_term[n] = sum_g w_scale[n][g] * (sum of the weight codes of row n in group g
//                                         - group_size * w_zero[n][g]);
// one wave per weight row, lanes over the row's groups.
__global__ __launch_bounds__(256) void weight_zero_term_kernel(const uint32_t *__restrict__ planes, int N, int KW, int bits,
                                                               int is_signed, const float *__restrict__ w_scale,
                                                               const float *__restrict__ w_zero, int group_size,
                                                               float *__restrict__ out)
{
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (n >= N)
        return; // whole waves leave; no barrier below
    const int wpg = group_size / 32, groups = KW / wpg;
    float t = 0.f;
    for (int gi = lane; gi < groups; gi += 64) {
        int sum = 0;
        for (int b = 0; b < bits; ++b) {
            int c = 0;
            for (int w = 0; w < wpg; ++w)
                c += __popc(planes[((size_t)b * N + n) * KW + gi * wpg + w]);
            sum += (is_signed && b == bits - 1) ? -(c << b) : (c << b);
        }
        const size_t idx = (size_t)n * groups + gi;
        t += w_scale[idx] * ((float)sum - (float)group_size * (w_zero ? w_zero[idx] : 0.f));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        t += __shfl_xor(t, o);
    if (lane == 0)
        out[n] = t;
}

hipError_t launch_weight_zero_term(const uint32_t *planes, int n, int k, int bits, int is_signed, const float *w_scale,
                                   const float *w_zero, int group_size, float *out, hipStream_t stream)
{
    hipLaunchKernelGGL(weight_zero_term_kernel, dim3((n + 3) / 4), dim3(256), 0, stream, planes, n, k / 32, bits,
                       is_signed, w_scale, w_zero, group_size, out);
    return hipGetLastError();
}

static int grid_for(size_t items)
{
    size_t blocks = (items + 255) / 256;
    if (blocks > 256 * 16)
        blocks = 256 * 16;
    if (blocks < 1)
        blocks = 1;
    return (int)blocks;
}

hipError_t launch_pack_i32(const int32_t *in, uint32_t *planes, int rows, int k, int bits,
                           hipStream_t stream)
{
    const size_t n_units = (size_t)rows * k / 8;
    hipLaunchKernelGGL(pack_i32_kernel, dim3(grid_for(n_units)), dim3(256), 0, stream,
                       reinterpret_cast<const int4 *>(in), planes, n_units, bits);
    return hipGetLastError();
}

hipError_t launch_pack_f16_tiled(const void *in, const float *scale, uint32_t *tiled, int rows, int k, int bits,
                                 hipStream_t stream)
{
    const size_t n_units = (size_t)rows * k / 8;
    hipLaunchKernelGGL(pack_f16_tiled_kernel<false>, dim3(grid_for(n_units)), dim3(256), 0, stream,
                       reinterpret_cast<const uint4 *>(in), scale, tiled, rows, k / 8, bits, 0);
    return hipGetLastError();
}

hipError_t launch_pack_f16_fp6(const void *in, const float *scale, uint32_t *records, int rows, int k, int bits, int is_signed,
                               hipStream_t stream)
{
    const size_t n_units = (size_t)rows * k / 8;
    hipLaunchKernelGGL(pack_f16_tiled_kernel<true>, dim3(grid_for(n_units)), dim3(256), 0, stream,
                       reinterpret_cast<const uint4 *>(in), scale, records, rows, k / 8, bits, is_signed);
    return hipGetLastError();
}

hipError_t launch_pack_f16(const void *in, const float *scale, uint32_t *planes, int rows, int k,
                           int bits, hipStream_t stream)
{
    const size_t n_units = (size_t)rows * k / 8;
    hipLaunchKernelGGL(pack_f16_kernel, dim3(grid_for(n_units)), dim3(256), 0, stream,
                       reinterpret_cast<const uint4 *>(in), scale, planes, n_units, bits);
    return hipGetLastError();
}

hipError_t launch_pack_u4(const uint32_t *in, uint32_t *planes, int rows, int k, int bits,
                          hipStream_t stream)
{
    const size_t n_words = (size_t)rows * k / 32;
    hipLaunchKernelGGL(pack_u4_kernel, dim3(grid_for(n_words)), dim3(256), 0, stream,
                       reinterpret_cast<const uint4 *>(in), planes, n_words, bits);
    return hipGetLastError();
}

} // namespace abq
