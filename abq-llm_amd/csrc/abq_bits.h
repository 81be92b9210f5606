// Bit-plane <-> byte helpers shared by the pack and GEMM kernels.
//
// Everything here is plain integer C++ so the same code compiles for the device (hipcc)
// and for the host (g++), where the unit tests drive it against the CPU oracle.
//
// Plane layout (engine/common/pack.cu:54-62 of the reference): element e of a group of 32
// consecutive K elements sits at bit (31 - e) of the plane word; plane b holds bit b.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define ABQ_HD __host__ __device__ __forceinline__
#else
#define ABQ_HD inline
#endif

namespace abq {

// One delta swap of a butterfly bit-matrix transpose: rows a (even) and b (odd) exchange
// the blocks selected by mask m / shift s.
ABQ_HD void delta_swap(uint32_t &a, uint32_t &b, uint32_t m, int s)
{
    uint32_t na = (a & m) | ((b << s) & ~m);
    uint32_t nb = ((a >> s) & m) | (b & ~m);
    a = na;
    b = nb;
}

// In-place transpose of the 8x8 bit matrices formed by r[0..7] (rows) and the 8 bit
// positions of each of the 4 byte lanes (columns).  After the call, byte c of r[s] has at
// bit j what bit (8c + s) of the old r[j] was.
ABQ_HD void transpose8x8x4(uint32_t (&r)[8])
{
    delta_swap(r[0], r[1], 0x55555555u, 1);
    delta_swap(r[2], r[3], 0x55555555u, 1);
    delta_swap(r[4], r[5], 0x55555555u, 1);
    delta_swap(r[6], r[7], 0x55555555u, 1);
    delta_swap(r[0], r[2], 0x33333333u, 2);
    delta_swap(r[1], r[3], 0x33333333u, 2);
    delta_swap(r[4], r[6], 0x33333333u, 2);
    delta_swap(r[5], r[7], 0x33333333u, 2);
    delta_swap(r[0], r[4], 0x0F0F0F0Fu, 4);
    delta_swap(r[1], r[5], 0x0F0F0F0Fu, 4);
    delta_swap(r[2], r[6], 0x0F0F0F0Fu, 4);
    delta_swap(r[3], r[7], 0x0F0F0F0Fu, 4);
}

// How a BITS-wide operand is laid into an int8 lane for the matrix cores.
//   kTop    signed operand: plane j goes to byte bit (8-BITS+j), so the MSB plane lands on the
//           int8 sign bit and the byte equals value * 2^(8-BITS) in two's complement.
//   kLow    unsigned operand of at most 7 bits: plane j goes to byte bit j.
//   kFlip   unsigned 8-bit operand: bit 7 is inverted, the byte reads as value - 128.
enum Int8Mode { kTop = 0, kLow = 1, kFlip = 2 };

template <int BITS, bool SIGNED> struct Int8ModeOf {
    static constexpr Int8Mode value = SIGNED ? kTop : (BITS == 8 ? kFlip : kLow);
};

// Expand BITS plane words (32 K elements) into 32 int8 values, as 8 dwords.
// out[s] byte c is the element at bit position (8c + s) of the plane words, i.e. element
// e = 31 - (8c + s) of the 32-group.  The element order does not depend on BITS or MODE, so
// an activation word and a weight word expanded by this routine pair up element by element.
template <int BITS, Int8Mode MODE> ABQ_HD void planes_to_int8(const uint32_t (&w)[BITS], uint32_t (&out)[8])
{
    static_assert(BITS >= 1 && BITS <= 8, "1..8 planes");
#pragma unroll
    for (int j = 0; j < 8; ++j)
        out[j] = 0u;
#pragma unroll
    for (int j = 0; j < BITS; ++j)
        out[MODE == kTop ? 8 - BITS + j : j] = w[j];
    if (MODE == kFlip)
        out[7] = ~out[7];
    transpose8x8x4(out);
}

// Sum of the unsigned values of the 32 elements held by BITS plane words.
template <int BITS> ABQ_HD int planes_value_sum(const uint32_t (&w)[BITS])
{
    int s = 0;
#pragma unroll
    for (int j = 0; j < BITS; ++j)
        s += __builtin_popcount(w[j]) << j;
    return s;
}

// 8x8 bit-matrix transpose of a 64-bit word (byte r, bit c) -> (byte c, bit r).
ABQ_HD uint64_t transpose8x8(uint64_t x)
{
    uint64_t t;
    t = (x ^ (x >> 7)) & 0x00AA00AA00AA00AAull;
    x = x ^ t ^ (t << 7);
    t = (x ^ (x >> 14)) & 0x0000CCCC0000CCCCull;
    x = x ^ t ^ (t << 14);
    t = (x ^ (x >> 28)) & 0x00000000F0F0F0F0ull;
    x = x ^ t ^ (t << 28);
    return x;
}

// ---- field-packed K tiles ------------------------------------------------------------------
//
// The LDS-staged MFMA kernels keep their operands in a second, library-private format whose
// unpacking to int8 costs one or two vector instructions per four elements instead of the
// bit-matrix transpose that plane words need.  A row's K tile of 128 elements is one record of
// BITS * 4 words; the element order inside a 32-element word-set is the one planes_to_int8
// produces ("expanded" dword s, byte c = element 31 - (8c + s)).  The BITS-bit pattern of an
// element is cut into fields, most significant first:
//     8 bits: one 8-bit field (the bytes themselves);
//     else  : a 4-bit, a 2-bit and a 1-bit field for every set bit of BITS (7 = 4+2+1, 6 = 4+2,
//             5 = 4+1, 3 = 2+1).
// A field of width f holds, per word-set, f words: word j carries in byte c, at bits
// [f*s, f*s+f), the field of the element at expanded dword (8/f)*j + s, byte c.  In the record
// the field of width f starts at word 4 * (BITS & ~(2f-1)) and its word-sets follow each other.
ABQ_HD constexpr uint32_t field_mask(int f) { return 0x01010101u * ((1u << f) - 1u); }
ABQ_HD constexpr int field_base(int bits, int f) { return bits & (f - 1); }             // lowest value bit of the field
ABQ_HD constexpr int field_word_offset(int bits, int f) { return 4 * (bits & ~(2 * f - 1)); }
// words of the wider fields in front of field f in a per-word-set list [4-bit: 4][2-bit: 2][1-bit: 1]
ABQ_HD constexpr int field_list_index(int bits, int f) { return bits & ~(2 * f - 1); }
// The routines below treat one field width at a time, as a template parameter: every trip count and register
// index is then a constant of the instantiation.  (Written as one loop over f = 4, 2, 1 with the inner trip
// count f, the compiler left the 6- and 7-bit cases rolled and indexed the register arrays at run time: the
// prefill kernel for those widths ran ten times slower than for 5 bits.)

// Expanded bytes (bit pattern in the low BITS bits of each byte) of one word-set -> its BITS
// field words, ordered [4-bit field: 4 words][2-bit field: 2 words][1-bit field: 1 word].
template <int BITS, int F> ABQ_HD void compress_one_field(const uint32_t (&e)[8], uint32_t (&out)[BITS])
{
    if constexpr ((BITS & F) != 0) {
        constexpr int per = 8 / F, idx = field_list_index(BITS, F);
#pragma unroll
        for (int j = 0; j < F; ++j) {
            uint32_t v = 0;
#pragma unroll
            for (int s = 0; s < per; ++s)
                v |= ((e[per * j + s] >> field_base(BITS, F)) & field_mask(F)) << (F * s);
            out[idx + j] = v;
        }
    }
}

template <int BITS> ABQ_HD void compress_fields(const uint32_t (&e)[8], uint32_t (&out)[BITS])
{
    static_assert(BITS >= 1 && BITS <= 8, "1..8 bits");
    if constexpr (BITS == 8) {
#pragma unroll
        for (int d = 0; d < 8; ++d)
            out[d] = e[d];
    } else {
        compress_one_field<BITS, 4>(e, out);
        compress_one_field<BITS, 2>(e, out);
        compress_one_field<BITS, 1>(e, out);
    }
}

// The reverse, fused with the placement in the int8 lane (MODE as for planes_to_int8).  `raw`
// holds the fields of WPT consecutive word-sets of one row, [4-bit field: 4*WPT words][2-bit:
// 2*WPT][1-bit: WPT] (or 8*WPT bytes-as-words for 8 bits); `ws` selects the word-set.
template <int BITS, int WPT, Int8Mode MODE, int F, int WS>
ABQ_HD void expand_one_field(const uint32_t (&raw)[BITS * WPT], uint32_t (&e)[8])
{
    if constexpr ((BITS & F) != 0) {
        constexpr int per = 8 / F, idx = field_list_index(BITS, F) * WPT;
        constexpr int t = field_base(BITS, F) + (MODE == kTop ? 8 - BITS : 0); // where the field lands in the byte
#pragma unroll
        for (int j = 0; j < F; ++j) {
            const uint32_t w = raw[idx + F * WS + j];
#pragma unroll
            for (int s = 0; s < per; ++s) {
                const int net = t - F * s;
                const uint32_t y = net >= 0 ? (w << (net & 31)) : (w >> ((-net) & 31));
                e[per * j + s] |= y & (field_mask(F) << t);
            }
        }
    }
}

template <int BITS, int WPT, Int8Mode MODE, int WS> ABQ_HD void expand_fields_of(const uint32_t (&raw)[BITS * WPT], uint32_t (&e)[8])
{
    static_assert(WS >= 0 && WS < WPT, "word-set of the list");
    if constexpr (BITS == 8) {
#pragma unroll
        for (int d = 0; d < 8; ++d)
            e[d] = raw[8 * WS + d] ^ (MODE == kFlip ? 0x80808080u : 0u);
    } else {
#pragma unroll
        for (int d = 0; d < 8; ++d)
            e[d] = 0u;
        expand_one_field<BITS, WPT, MODE, 4, WS>(raw, e);
        expand_one_field<BITS, WPT, MODE, 2, WS>(raw, e);
        expand_one_field<BITS, WPT, MODE, 1, WS>(raw, e);
    }
}

// the same with the word-set as an argument (0 <= ws < WPT <= 4)
template <int BITS, int WPT, Int8Mode MODE>
ABQ_HD void expand_fields(const uint32_t (&raw)[BITS * WPT], int ws, uint32_t (&e)[8])
{
    static_assert(WPT >= 1 && WPT <= 4, "at most four word-sets in a list");
    if (WPT == 1 || ws == 0)
        expand_fields_of<BITS, WPT, MODE, 0>(raw, e);
    else if (WPT == 2 || ws == 1)
        expand_fields_of<BITS, WPT, MODE, (WPT > 1 ? 1 : 0)>(raw, e);
    else if (WPT == 3 || ws == 2)
        expand_fields_of<BITS, WPT, MODE, (WPT > 2 ? 2 : 0)>(raw, e);
    else
        expand_fields_of<BITS, WPT, MODE, (WPT > 3 ? 3 : 0)>(raw, e);
}

// Sum of the four bytes of every dword of an expanded word-set (values fed unsigned, before
// any kFlip inversion).
ABQ_HD int expanded_byte_sum(const uint32_t (&e)[8])
{
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t s = 0;
#pragma unroll
    for (int d = 0; d < 8; ++d)
        s = __builtin_amdgcn_sad_u8(e[d], 0u, s); // sum of |byte - 0| over the four bytes
    return (int)s;
#else
    int s = 0;
    for (int d = 0; d < 8; ++d)
        s += (int)((e[d] & 0xFFu) + ((e[d] >> 8) & 0xFFu) + ((e[d] >> 16) & 0xFFu) + (e[d] >> 24));
    return s;
#endif
}

// Eight consecutive K elements (low 8 bits of each used) -> eight plane bytes.
// Byte b of the result is the 8-bit slice of plane b covering these elements, first
// element at the byte's bit 7 (the plane words are MSB first).
ABQ_HD uint64_t eight_values_to_plane_bytes(const int (&v)[8])
{
    uint64_t x = 0;
#pragma unroll
    for (int c = 0; c < 8; ++c)
        x |= (uint64_t)((uint32_t)v[c] & 0xFFu) << (8 * (7 - c));
    return transpose8x8(x);
}

// Multiplier of the popcount of (activation plane i AND weight plane j):
// +/- 2^(i+j), negative when exactly one of the two is the MSB plane of a signed operand
// (engine/test_any_mma.cu:64-68 and engine/mma_any/aq_bmma_kernel.h:549-561 of the reference).
ABQ_HD int plane_pair_weight(int i, int j, int x_bits, int w_bits, bool is_signed)
{
    int mag = 1 << (i + j);
    bool neg = is_signed && ((i == x_bits - 1) != (j == w_bits - 1));
    return neg ? -mag : mag;
}

// Nibble-packed input word (8 elements, first element in the top nibble) -> for plane b the
// 8-bit slice, first element at bit 7 (engine/common/pack.cu:26-40 of the reference).
ABQ_HD uint32_t nibble_word_plane_byte(uint32_t word, int b)
{
    uint32_t y = (word >> b) & 0x11111111u; // bit 4t <- bit b of nibble t (t = 7 - element)
    y = (y | (y >> 3)) & 0x03030303u;
    y = (y | (y >> 6)) & 0x000F000Fu;
    y = (y | (y >> 12)) & 0xFFu;
    return y;
}

} // namespace abq
