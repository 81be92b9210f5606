// abq_convert_weights: quantise one linear layer's weights and write them as a packed weight
// file (abq_weight_file.h), optionally also as the headerless plane dump the reference's
// FasterTransformer loader reads.
//
//   abq_convert_weights IN.bin N K BITS GROUP_SIZE {sym|asym} OUT.abqw [--fp16] [--ft-bin OUT.bin] [--bit-balance]
//
// IN.bin: row-major [N][K] float32 (or fp16 with --fp16), the layout of torch's linear.weight.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "abq_weight_file.h"

static float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { // subnormal: renormalise
            int e = -1;
            do {
                ++e;
                man <<= 1;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

int main(int argc, char **argv)
{
    if (argc < 8) {
        printf("Usage: ./abq_convert_weights IN.bin N K BITS GROUP_SIZE {sym|asym} OUT.abqw [--fp16] [--ft-bin OUT.bin] [--bit-balance]\n");
        return 2;
    }
    const std::string in = argv[1], mode = argv[6], out = argv[7];
    const uint32_t n = (uint32_t)atoi(argv[2]), k = (uint32_t)atoi(argv[3]), bits = (uint32_t)atoi(argv[4]),
                   group = (uint32_t)atoi(argv[5]);
    bool fp16 = false, bit_balance = false;
    std::string ft_bin;
    for (int i = 8; i < argc; ++i) {
        if (!strcmp(argv[i], "--fp16"))
            fp16 = true;
        else if (!strcmp(argv[i], "--ft-bin") && i + 1 < argc)
            ft_bin = argv[++i];
        else if (!strcmp(argv[i], "--bit-balance"))
            bit_balance = true; // the reference's default for asymmetric 1- and 2-bit weights: 2^BITS + 1 levels, BITS + 1 planes
    }
    if (mode != "sym" && mode != "asym") {
        printf("[ABQ][Error] mode must be sym or asym\n");
        return 2;
    }
    const size_t count = (size_t)n * k;
    std::vector<float> w(count);
    FILE *f = fopen(in.c_str(), "rb");
    if (!f) {
        printf("[ABQ][Error] cannot open %s\n", in.c_str());
        return 1;
    }
    bool ok;
    if (fp16) {
        std::vector<uint16_t> h(count);
        ok = fread(h.data(), 2, count, f) == count;
        for (size_t i = 0; ok && i < count; ++i)
            w[i] = half_to_float(h[i]);
    } else {
        ok = fread(w.data(), 4, count, f) == count;
    }
    ok = ok && fgetc(f) == EOF;
    fclose(f);
    if (!ok) {
        printf("[ABQ][Error] %s does not hold exactly %u x %u %s values\n", in.c_str(), n, k, fp16 ? "fp16" : "float32");
        return 1;
    }
    ABQWeightBlob blob;
    std::string err;
    if (!abq_quantize_weights(w.data(), n, k, bits, mode == "sym", group, &blob, &err, bit_balance) ||
        !abq_weight_file_write(out, blob, &err) || (!ft_bin.empty() && !abq_weight_file_write_ft_bin(ft_bin, blob, &err))) {
        printf("[ABQ][Error] %s\n", err.c_str());
        return 1;
    }
    printf("wrote %s: W%u %s%s, %u x %u, group %u, %u planes, %zu plane bytes\n", out.c_str(), bits, mode.c_str(),
           bit_balance ? " (bit balance)" : "", n, k, group, blob.info.bits, blob.planes.size() * 4);
    return 0;
}
