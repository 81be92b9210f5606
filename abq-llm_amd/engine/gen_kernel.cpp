// Tile search-space generator (host only).
//
// Same command line and output format as the reference's engine/gen_kernel.cpp:24-157:
//     gen_kernel X_BITS W_BITS SIGNED K_STAGE [--space gfx950|sm80] [--format macro|variants]
// prints one "AQ_INSTANTIATE_FUN(AqBMMA, ...);" line per tile configuration, preceded by a
// comment line per tile shape.
//
//   --space gfx950 (default)  the native MI355X space: VALU-popcount tiles (MMA 1x1x128), int8-MFMA
//                             tiles (MMA 16x16x64 and 32x32x32) and FP6-MFMA tiles, bounded by what one
//                             CDNA4 compute unit offers (wave64, 512 VGPRs per lane at one wave
//                             per SIMD, 160 KiB LDS, 1024 threads per workgroup).
//   --space sm80              the reference's own rules, restated; its output is compared with
//                             the reference generator and with the tile lists the reference
//                             ships (aq_bmma_impl/aq_bmma_w{2a8,3a3,5a5,7a7}.h).
//   --format variants         (gfx950 only) prints the MFMA part as V(MI,TM,TN,WM,WN,WK) lines,
//                             the form csrc/abq_mfma_variants.inc is kept in.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <set>
#include <string>
#include <tuple>
#include <vector>

namespace {

struct Tile {
    int bm, bn, bk;
    int wm, wn, wk;
    int mm, mn, mk;
    int x_waves, w_waves;
    std::vector<int> stages;
};

void print_tile(const Tile &t, int x_bits, int w_bits, bool is_signed)
{
    std::printf("// cta<%d,%d,%d> warp<%d,%d,%d> mma<%d,%d,%d>   WARPS[%dx%d]\n", t.bm, t.bn, t.bk,
                t.wm, t.wn, t.wk, t.mm, t.mn, t.mk, t.x_waves, t.w_waves);
    for (int s : t.stages)
        std::printf("AQ_INSTANTIATE_FUN(%s, %d, %d, %s, %d, %d, %d, %d, %d, %d, %d, %d, %d, %d);\n",
                    "AqBMMA", x_bits, w_bits, is_signed ? "true" : "false", t.bm, t.bn, t.bk, t.wm,
                    t.wn, t.wk, t.mm, t.mn, t.mk, s);
}

// ------------------------------------------------------------------------------------------
// sm80: the reference's rules (engine/gen_kernel.cpp:36-149), written as a list of predicates.
// ------------------------------------------------------------------------------------------
std::vector<Tile> enumerate_sm80(int x_bits, int w_bits, int k_stages)
{
    const size_t kSmemPerSm = 102400, kSmemOptIn = 101376; // gen_kernel.cpp:36-37
    const int kRegsPerThread = 255;                        // :38
    auto allowed_block_m = [&](int bm) {                   // whitelist BMS, :40-42
        switch (x_bits) {
        case 2: return bm == 4 || bm == 8;
        case 3: return bm == 2 || bm == 8;
        case 4: return bm == 2 || bm == 4 || bm == 8;
        case 5: return bm == 1 || bm == 8;
        case 6: return bm == 1 || bm == 4 || bm == 8;
        case 7: return bm == 1 || bm == 8;
        case 8: return bm == 1 || bm == 4 || bm == 8;
        default: return false;
        }
    };
    auto smem_fits = [&](size_t bytes) { return bytes < kSmemPerSm && bytes < kSmemOptIn; };

    std::vector<Tile> out;
    std::set<std::tuple<int, int, int, int, int, int>> seen;
    for (int bk : { 256, 384, 512 }) {                      // :44, "BK = 128 is inefficient"
        for (int xw = 1; xw <= 32; xw *= 2) {
            for (int ww = 1; ww <= 32; ww *= 2) {
                const int waves = xw * ww;
                if (waves > 32 || waves == 1 || waves >= 8) // :50-55
                    continue;
                for (int wm = 8; wm <= 64; wm += 8) {
                    for (int wn = 8; wn <= 128; wn += 8) {
                        const bool wide = wm % 16 == 0;     // :61-64
                        const int mm = wide ? 16 : 8, mn = 8, mk = wide ? 256 : 128;
                        if (bk % mk != 0)
                            continue;
                        const int tiles_m = wm / mm, tiles_n = wn / mn;
                        const int regs = tiles_m * mm * mk / 1024 + tiles_n * mn * mk / 1024 +
                                         tiles_m * tiles_n * mm * mn / 32; // :71-75
                        if (regs > kRegsPerThread)
                            continue;
                        const int bm = xw * tiles_m * mm / x_bits; // :77-78
                        const int bn = ww * tiles_n * mn / w_bits;
                        if (bm > 8 || !allowed_block_m(bm))
                            continue;
                        if (bn < 32 || bn % 16 != 0)
                            continue;
                        if (bn > mk && bn % mk != 0)
                            continue;
                        const int skew = (w_bits * bn) % 16 == 0 ? 8 : 0; // :100
                        const size_t stage_bytes = (size_t)bm * bk * x_bits / 8 + (size_t)bn * bk * w_bits / 8;
                        const size_t out_bytes = (size_t)(mm * tiles_m * xw) * (mn * tiles_n * ww + skew) * sizeof(int);
                        const size_t max_stages = out_bytes > 2 * stage_bytes ? out_bytes / stage_bytes : (size_t)k_stages;
                        if (!smem_fits(std::max(2 * stage_bytes, out_bytes)))
                            continue;
                        if (!seen.insert(std::make_tuple(bm, bn, bk, wm, wn, mk)).second)
                            continue;
                        Tile t{ bm, bn, bk, wm, wn, mk, mm, mn, mk, xw, ww, {} };
                        for (size_t s = 2; s <= max_stages; ++s)
                            if (smem_fits(std::max(s * stage_bytes, out_bytes)))
                                t.stages.push_back((int)s);
                        out.push_back(t);
                    }
                }
            }
        }
    }
    return out;
}

// ------------------------------------------------------------------------------------------
// gfx950: the native space.
// ------------------------------------------------------------------------------------------
struct MfmaVariant {
    int mi, tm, tn, wm, wn, wk;
};

// Matrix-core tiles.  A wave holds TM x TN accumulator tiles of MI x MI int32 and, double
// buffered, the plane words of TM activation rows and TN weight rows (4 words per plane).
std::vector<MfmaVariant> enumerate_mfma(int x_bits, int w_bits)
{
    const int kVgprBudget = 448;      // of 512, the rest is addressing and expansion temporaries
    const int kLdsBytes = 160 * 1024; // per compute unit
    const int kMaxWaves = 16;         // 1024 threads
    std::vector<MfmaVariant> out;
    for (int mi : { 16, 32 }) {
        const int acc = mi == 16 ? 4 : 16;
        for (int tm = 1; tm <= 4; tm *= 2) {
            for (int tn = 1; tn <= 4; tn *= 2) {
                const int regs = tm * tn * acc + 2 * 4 * (tm * x_bits + tn * w_bits) + 8 * (tm + tn);
                if (regs > kVgprBudget)
                    continue;
                for (int wm = 1; wm <= 4; wm *= 2) {
                    for (int wn = 1; wn <= 4; wn *= 2) {
                        for (int wk = 1; wk <= 8; wk *= 2) {
                            const int waves = wm * wn * wk;
                            if (waves < 2 || waves > kMaxWaves)
                                continue;
                            const long lds = (long)wm * wn * (wk - 1) * (tm * tn * acc + tm + tn) * 256;
                            if (lds > kLdsBytes / 2)
                                continue;
                            // 16-row tiles serve decode: one tile along M, K split over the waves.
                            // 32-row tiles serve prefill: waves tile M x N, no K split.
                            if (mi == 16 && (tm != 1 || wm != 1 || wk < 2 || tn > 2 || wn > 2 || waves < 4 || waves > 8))
                                continue;
                            if (mi == 32 && (wk != 1 || wm != 2 || wn != 2 || tm > tn || tn > 2))
                                continue;
                            out.push_back({ mi, tm, tn, wm, wn, wk });
                        }
                    }
                }
            }
        }
    }
    return out;
}

std::vector<Tile> enumerate_gfx950(int x_bits, int w_bits, bool is_signed)
{
    std::vector<Tile> out;
    // VALU popcount: MT activation rows per workgroup, LPR lanes per weight row (16, 32, 64), eight waves;
    // NSTAGE = passes of a lane whose loads are in flight together (1 or 3).
    for (int d : { 1, 3 }) {
        for (int mt : { 1, 2, 4 }) {
            for (int lpr : { 16, 32, 64 }) {
                const int rows = 64 / lpr;
                out.push_back(Tile{ mt, 8 * rows, lpr * 128, mt, rows, lpr * 128, 1, 1, 128, 1, 8, { d } });
            }
        }
    }
    // Decode kernel: 16-row MFMA tiles, activations expanded once per workgroup into LDS
    // (NSTAGE = 3), NW waves per workgroup splitting K.
    for (int nw : { 4, 8, 16 })
        out.push_back(Tile{ 16, 16, 512 * nw, 16, 16, 512, 16, 16, 64, 1, nw, { 3 } });
    // the same with steps of 256 K elements (short K spread over all waves)
    out.push_back(Tile{ 16, 16, 256 * 16, 16, 16, 256, 16, 16, 64, 1, 16, { 3 } });
    for (const MfmaVariant &v : enumerate_mfma(x_bits, w_bits)) {
        const int stepk = (64 / v.mi) * 4 * 32;
        out.push_back(Tile{ v.mi * v.tm * v.wm, v.mi * v.tn * v.wn, stepk * v.wk, v.mi * v.tm, v.mi * v.tn,
                            stepk, v.mi, v.mi, 1024 / v.mi, v.wm, v.wn * v.wk, { 2 } });
    }
    // LDS-staged prefill kernel on the K-tiled layout (NSTAGE = 4): 2 x 2 waves, TM x TN MFMA
    // tiles of 32 x 32 per wave, K tile 128.  Double-buffered int8 tiles must fit 160 KiB of LDS.
    const int tiled[][2] = { { 4, 4 }, { 2, 4 }, { 2, 2 }, { 2, 1 }, { 1, 1 } };
    for (const auto &t : tiled) {
        const int bm = 64 * t[0], bn = 64 * t[1];
        if (2 * (bm + bn) * 144 + (bm + bn) * 4 > 160 * 1024)
            continue;
        out.push_back(Tile{ bm, bn, 128, 32 * t[0], 32 * t[1], 128, 32, 32, 32, 2, 2, { 4 } });
    }
    // the same with 64-element K stages (half the LDS per stage: two workgroups per compute unit
    // for the 128 x 256 tile)
    // larger workgroups (4 x 2 and 4 x 4 waves of 64 x 64): less L2 -> L1 traffic per MFMA
    out.push_back(Tile{ 256, 128, 128, 64, 64, 128, 32, 32, 32, 4, 2, { 4 } });
    out.push_back(Tile{ 256, 256, 128, 64, 64, 128, 32, 32, 32, 4, 4, { 4 } });
    out.push_back(Tile{ 256, 256, 128, 64, 128, 128, 32, 32, 32, 4, 2, { 4 } });
    // activations wider than the weights, both of a single field (2, 4, 8 bits): 128 x 256 on the staged
    // kernel, eight waves of 64 x 64 (2 along M, 4 along N)
    {
        const bool field = (x_bits == 2 || x_bits == 4 || x_bits == 8) && (w_bits == 2 || w_bits == 4 || w_bits == 8);
        if (field && x_bits > w_bits && (is_signed || x_bits < 8))
            out.push_back(Tile{ 128, 256, 128, 64, 64, 128, 32, 32, 32, 2, 4, { 4 } });
        // small grids on the staged kernel: two groups of waves that split K inside the workgroup (64 x 64 and
        // 128 x 64), and a 64 x 128 tile, plain and split, where an activation row is the longer record
        if (field && (is_signed || (x_bits < 8 && w_bits < 8))) {
            out.push_back(Tile{ 64, 64, 256, 32, 32, 128, 32, 32, 32, 2, 4, { 4 } });
            out.push_back(Tile{ 128, 64, 256, 64, 32, 128, 32, 32, 32, 2, 4, { 4 } });
            if (x_bits + w_bits < 16) // three stages of two K tiles of 128 x 128 fit the LDS
                out.push_back(Tile{ 128, 128, 256, 64, 64, 128, 32, 32, 32, 2, 4, { 4 } });
        }
        if (field && x_bits > w_bits && (is_signed || x_bits < 8)) {
            out.push_back(Tile{ 64, 128, 128, 32, 64, 128, 32, 32, 32, 2, 2, { 4 } });
            out.push_back(Tile{ 64, 128, 256, 32, 64, 128, 32, 32, 32, 2, 4, { 4 } });
        }
    }
    const int half[][2] = { { 2, 4 }, { 2, 2 } };
    for (const auto &t : half)
        out.push_back(Tile{ 64 * t[0], 64 * t[1], 64, 32 * t[0], 32 * t[1], 64, 32, 32, 32, 2, 2, { 4 } });
    // FP6 matrix-core kernel (NSTAGE = 5, MMA 32x32x64): operands that are E2M3 numbers, i.e. unsigned
    // of at most 4 bits or signed of at most 5; { TM, TN, waves along M, waves along N }
    const int lim = is_signed ? 5 : 4;
    if (x_bits <= lim && w_bits <= lim) {
        const int fp6[][4] = { { 2, 2, 4, 2 }, { 4, 2, 2, 2 }, { 2, 2, 2, 2 }, { 2, 1, 2, 2 }, { 1, 1, 2, 2 } };
        for (const auto &t : fp6)
            out.push_back(Tile{ 32 * t[0] * t[2], 32 * t[1] * t[3], 128, 32 * t[0], 32 * t[1], 128, 32, 32, 64, t[2], t[3], { 5 } });
    }
    // Decode kernel on K-tiled operands (NSTAGE = 6).  Weights of one field (2, 4, 8 bits; activations of several
    // fields reach it as records of the next single-field width): { waves, weight loads in flight per wave, 16-row
    // tiles per workgroup }, a load covers 512 / W_BITS elements of K.  Weights of several fields (3, 5, 6, 7 bits,
    // read field by field): { waves, loads in flight }, warp K in the name = 128 x loads.
    {
        const bool w_field = w_bits == 2 || w_bits == 4 || w_bits == 8;
        if (w_field && x_bits >= w_bits) {
            const int dt[][3] = { { 16, 1, 1 }, { 16, 3, 1 }, { 8, 2, 1 }, { 16, 1, 3 }, { 8, 1, 2 }, { 8, 2, 2 }, { 16, 1, 2 } };
            const int stepk = 512 / w_bits;
            for (const auto &v : dt)
                out.push_back(Tile{ 16, 16 * v[2], stepk * v[1] * v[0], 16, 16 * v[2], stepk * v[1], 16, 16, 64, 1, v[0], { 6 } });
        } else if (!w_field && x_bits >= w_bits) {
            const int df[][2] = { { 16, 2 }, { 16, 4 }, { 8, 4 } };
            for (const auto &v : df)
                out.push_back(Tile{ 16, 16, 128 * v[1] * v[0], 16, 16, 128 * v[1], 16, 16, 64, 1, v[0], { 6 } });
        }
    }
    return out;
}

} // namespace

int main(int argc, char **argv)
{
    if (argc < 5) {
        std::printf("Usage: ./gen_kernel X_BITS W_BITS SIGNED K_STAGE [--space gfx950|sm80] [--format macro|variants]\n");
        return -1;
    }
    const int x_bits = std::atoi(argv[1]);
    const int w_bits = std::atoi(argv[2]);
    const bool is_signed = std::atoi(argv[3]) == 1;
    const int k_stages = std::atoi(argv[4]);
    std::string space = "gfx950", format = "macro";
    for (int i = 5; i + 1 < argc; i += 2) {
        if (!std::strcmp(argv[i], "--space"))
            space = argv[i + 1];
        else if (!std::strcmp(argv[i], "--format"))
            format = argv[i + 1];
    }
    if (format == "variants") {
        for (const MfmaVariant &v : enumerate_mfma(x_bits, w_bits))
            std::printf("V(%d, %d, %d, %d, %d, %d)\n", v.mi, v.tm, v.tn, v.wm, v.wn, v.wk);
        return 0;
    }
    std::printf("////// W%dA%d %s\n", w_bits, x_bits, is_signed ? "int" : "uint");
    const std::vector<Tile> tiles = space == "sm80" ? enumerate_sm80(x_bits, w_bits, k_stages)
                                                    : enumerate_gfx950(x_bits, w_bits, is_signed);
    for (const Tile &t : tiles)
        print_tile(t, x_bits, w_bits, is_signed);
    return 0;
}
