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

extern "C" {

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
