// Host build of the bit helpers the HIP kernels use (abq-llm_amd/csrc/abq_bits.h), exported
// with C linkage so the CPU tests can drive them against the oracle.  Test code only.
#include <stdint.h>

#include "abq_bits.h"

using namespace abq;

template <int BITS> static void expand(int mode, const uint32_t *w, uint32_t *out)
{
    uint32_t in[BITS], o[8];
    for (int i = 0; i < BITS; ++i)
        in[i] = w[i];
    if (mode == kTop)
        planes_to_int8<BITS, kTop>(in, o);
    else if (mode == kLow)
        planes_to_int8<BITS, kLow>(in, o);
    else
        planes_to_int8<BITS, kFlip>(in, o);
    for (int i = 0; i < 8; ++i)
        out[i] = o[i];
}

// one word-set through the field-packed route: planes -> expanded (low) bytes -> fields -> int8
template <int BITS> static void via_fields(int mode, const uint32_t *w, uint32_t *fields, uint32_t *o, int *sum)
{
    uint32_t a[BITS], e[8], f[BITS], r[8];
    for (int i = 0; i < BITS; ++i)
        a[i] = w[i];
    planes_to_int8<BITS, kLow>(a, e);
    compress_fields<BITS>(e, f);
    for (int i = 0; i < BITS; ++i)
        fields[i] = f[i];
    if (mode == kTop)
        expand_fields<BITS, 1, kTop>(f, 0, r);
    else if (mode == kLow)
        expand_fields<BITS, 1, kLow>(f, 0, r);
    else
        expand_fields<BITS, 1, kFlip>(f, 0, r);
    for (int i = 0; i < 8; ++i)
        o[i] = r[i];
    uint32_t plain[8];
    expand_fields<BITS, 1, kLow>(f, 0, plain);
    *sum = expanded_byte_sum(plain);
}

extern "C" {

// words: [n][bits] plane words; fields: [n][bits] field words; out: [n][8] dwords; sums: [n]
void shim_via_fields(int bits, int mode, const uint32_t *words, uint32_t *fields, uint32_t *out, int *sums, long n)
{
    for (long i = 0; i < n; ++i) {
        const uint32_t *w = words + i * bits;
        uint32_t *f = fields + i * bits, *o = out + i * 8;
        switch (bits) {
        case 1: via_fields<1>(mode, w, f, o, sums + i); break;
        case 2: via_fields<2>(mode, w, f, o, sums + i); break;
        case 3: via_fields<3>(mode, w, f, o, sums + i); break;
        case 4: via_fields<4>(mode, w, f, o, sums + i); break;
        case 5: via_fields<5>(mode, w, f, o, sums + i); break;
        case 6: via_fields<6>(mode, w, f, o, sums + i); break;
        case 7: via_fields<7>(mode, w, f, o, sums + i); break;
        case 8: via_fields<8>(mode, w, f, o, sums + i); break;
        }
    }
}

// words: [n][bits] plane words of n 32-groups; out: [n][8] dwords = 32 int8 each
void shim_planes_to_int8(int bits, int mode, const uint32_t *words, uint32_t *out, long n)
{
    for (long i = 0; i < n; ++i) {
        const uint32_t *w = words + i * bits;
        uint32_t *o = out + i * 8;
        switch (bits) {
        case 1: expand<1>(mode, w, o); break;
        case 2: expand<2>(mode, w, o); break;
        case 3: expand<3>(mode, w, o); break;
        case 4: expand<4>(mode, w, o); break;
        case 5: expand<5>(mode, w, o); break;
        case 6: expand<6>(mode, w, o); break;
        case 7: expand<7>(mode, w, o); break;
        case 8: expand<8>(mode, w, o); break;
        }
    }
}

uint64_t shim_eight_values_to_plane_bytes(const int *v)
{
    int a[8];
    for (int i = 0; i < 8; ++i)
        a[i] = v[i];
    return eight_values_to_plane_bytes(a);
}

uint32_t shim_nibble_word_plane_byte(uint32_t word, int b) { return nibble_word_plane_byte(word, b); }

int shim_plane_pair_weight(int i, int j, int x_bits, int w_bits, int is_signed)
{
    return plane_pair_weight(i, j, x_bits, w_bits, is_signed != 0);
}

int shim_int8_mode(int bits, int is_signed) { return is_signed ? kTop : (bits == 8 ? kFlip : kLow); }
}
