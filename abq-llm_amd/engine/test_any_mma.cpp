// Autotune / benchmark harness: the MI355X counterpart of the reference's
// engine/test_any_mma.cu (main, :86-272) and engine/test/test_mma/test_mma.h (benchmark, TEST,
// :21-160).
//
//     test_any_mma M N K X_BITS W_BITS SIGNED [--repeat R] [--warmup W] [--rotate-mib MiB]
//                  [--stream] [--only SUBSTR] [--seed S] [--read-floor] [--zero-operands]
//                  [--tuning FILE] [--tuning-out FILE] [--no-builtin-tuning]
//
// Like the reference it builds random operands, packs them on the GPU, computes the expected
// result on the CPU, then runs EVERY tile configuration of the bit combination, checks each
// result for exact equality and prints one line per configuration
//     <arch> <WxAy int|uint> BM BN BK WM WN WK MM MN MK NSTAGE packing _ (us) exec _ (us)
//     _ TOPS | _ B-TOPS | PASSED|ERROR|FAILED
// followed by "The best kernel config is ... with ... TOPS".  TOPS = 2*M*N*K / t and
// B-TOPS = TOPS * X_BITS * W_BITS as in engine/test/test_mma/test_mma_w2a8.cu:37-38.
//
// Differences that matter on this hardware:
//  * the search space is the library's native gfx950 tile list (abq_native_config_*), plus the
//    library's own default choice as the last line;
//  * weights rotate through --rotate-mib of distinct buffers (default 512) so that the 256 MB
//    Infinity Cache cannot serve them; all buffers hold the same data, so one CPU result
//    checks them all;
//  * the timed loop is replayed from a HIP graph unless --stream is given, so the host launch
//    rate does not bound the figure; in addition to the roofline fractions it prints
//    (HBM 8 TB/s on the packed bytes, int8 MFMA 5 POP/s on 2*M*N*K);
//  * kernels on the K-tiled layout (NSTAGE 4) get weights converted once before the timed loop
//    (part of weight preparation, like packing) and convert the activations inside every call;
//    the decode kernel of that layout (NSTAGE 6) gets the activations K-tiled as well, which is how
//    the quantising kernel hands them over, and for M <= 16 a last line times the library's own
//    choice on such operands;
//  * --read-floor adds two lines timed the same way (same rotation, same graph replay): a kernel
//    that does nothing, and one that reads the packed weights once with 16-byte loads and computes
//    nothing: the floor of one launch over that many bytes;
//  * the sweep's result is consumed: --tuning-out FILE appends the fastest tile of each operand layout (planes,
//    K-tiled records, FP6 records) as "<kernel name> M N K 0 TOPS" lines, the format abq_tuning_load reads and the
//    library's compiled-in table (engine/tuning_mi355x.txt) is made of; --tuning FILE loads such a file first and
//    --no-builtin-tuning switches the compiled-in entries off, so that the "library default" line, which prepares
//    the weights in the layout abq_preferred_weight_layout names (above 16 rows) and lets the library pick the tile,
//    shows what the table, or the rules alone, make of the shape;
//  * inputs come from std::mt19937_64 with a fixed seed instead of unseeded rand(); --zero-operands makes every
//    code zero instead: the same instructions on operands that toggle no bits, i.e. what the kernels' time owes
//    to the clock the chip sustains on real data.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "abq_gemm.h"
#include "abq_probe.h" // measurement probes, not part of the library's interface

#define HIP_OK(x)                                                                        \
    do {                                                                                 \
        hipError_t e_ = (x);                                                             \
        if (e_ != hipSuccess) {                                                          \
            std::fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(1);                                                                \
        }                                                                                \
    } while (0)

namespace {

// Untimed replays of a graph before its timed one: the first launch uploads the graph, and a chip that has idled
// (behind a CPU check, or at the start of a sweep) takes tens of milliseconds of load to raise its clock; without
// them the tiles timed first in a sweep measured up to 17 % slower than the same tile timed last.
void warm_replays(hipGraphExec_t ge, hipStream_t stream)
{
    const auto t0 = std::chrono::steady_clock::now();
    do {
        if (hipGraphLaunch(ge, stream) != hipSuccess || hipStreamSynchronize(stream) != hipSuccess)
            return;
    } while (std::chrono::steady_clock::now() - t0 < std::chrono::milliseconds(50));
}


// Expected result, computed from the packed planes the way compute_ref does
// (engine/test_any_mma.cu:58-84) but with one popcount per word pair.
void expected_result(const std::vector<uint32_t> &w, const std::vector<uint32_t> &x, std::vector<int> &d, int M,
                     int N, int K, int w_bits, int x_bits, bool is_signed)
{
    const long KW = K / 32;
#pragma omp parallel for collapse(2) schedule(static)
    for (int m = 0; m < M; ++m) {
        for (int n = 0; n < N; ++n) {
            long acc = 0;
            for (int xb = 0; xb < x_bits; ++xb) {
                for (int wb = 0; wb < w_bits; ++wb) {
                    const uint32_t *xr = &x[((long)xb * M + m) * KW];
                    const uint32_t *wr = &w[((long)wb * N + n) * KW];
                    long cnt = 0;
                    for (long k = 0; k < KW; ++k)
                        cnt += __builtin_popcount(xr[k] & wr[k]);
                    const bool neg = is_signed && ((xb == x_bits - 1) != (wb == w_bits - 1));
                    acc += (neg ? -cnt : cnt) << (xb + wb);
                }
            }
            d[(long)m * N + n] = (int)acc;
        }
    }
}

struct Timing {
    float exec_us = 0, pack_us = 0;
    int status = -1; // 0 PASSED, -1 ERROR, -2 FAILED (test_mma.h:114-159)
};

// --mfma-ceiling: what the matrix cores sustain in a register-only loop (abq_probe_launch), on constant operand
// bits and on random ones, int8 and FP6: launches of about 30 ms so that clocks settle, the best of three.
int matrix_core_ceiling(hipStream_t stream)
{
    int dev = 0, cus = 0;
    HIP_OK(hipGetDevice(&dev));
    HIP_OK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    std::mt19937 rng(1);
    std::vector<uint32_t> h(2048);
    uint32_t *d;
    HIP_OK(hipMalloc(&d, h.size() * 4));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    const size_t n = 1u << 19;
    for (int kind : { ABQ_PROBE_MFMA_I8, ABQ_PROBE_MFMA_FP6 })
        for (int random = 0; random < 2; ++random) {
            // FP6: six dwords of a lane's eight hold 32 codes; constant = every code 0b001000 (1.0), i8: every byte 1
            for (auto &v : h)
                v = random ? (uint32_t)rng() : (kind == ABQ_PROBE_MFMA_FP6 ? 0x20820820u : 0x01010101u);
            HIP_OK(hipMemcpy(d, h.data(), h.size() * 4, hipMemcpyHostToDevice));
            float best = 1e30f;
            for (int rep = 0; rep < 4; ++rep) {
                HIP_OK(hipEventRecord(e0, stream));
                if (abq_probe_launch(kind, d, n, stream) != ABQ_OK)
                    return -1;
                HIP_OK(hipEventRecord(e1, stream));
                HIP_OK(hipStreamSynchronize(stream));
                float ms;
                HIP_OK(hipEventElapsedTime(&ms, e0, e1));
                if (rep)
                    best = std::min(best, ms);
            }
            const double ops = 2.0 * cus * 4 * (double)n * (kind == ABQ_PROBE_MFMA_FP6 ? 131072.0 : 65536.0);
            std::printf("matrix-core ceiling: %s, %s operand bits: %.1f ms per launch, %.2f P%s/s on %d compute units\n",
                        kind == ABQ_PROBE_MFMA_FP6 ? "v_mfma_f32_32x32x64_f8f6f4 (E2M3)" : "v_mfma_i32_32x32x32_i8",
                        random ? "random" : "constant", best, ops / (best * 1e-3) / 1e15, kind == ABQ_PROBE_MFMA_FP6 ? "FLOP" : "OP", cus);
        }
    (void)hipFree(d);
    return 0;
}

double half_bits_to_double(uint16_t h)
{
    const int e = (h >> 10) & 31, f = h & 1023;
    const double v = e == 0 ? std::ldexp((double)f, -24) : e == 31 ? (f ? NAN : INFINITY) : std::ldexp((double)(f | 1024), e - 25);
    return (h & 0x8000) ? -v : v;
}

// --group G [--fp6]: every tile of the kernels that carry group scales (the dequantising epilogue: weight scales
// and zero points per G elements of K, per-token activation scales, fp16 out), on prepared operands (K-tiled, or
// FP6 records with --fp6), plus the library's own choice.  Results are checked on up to eight rows against a
// double-precision loop over the dequantised operands (1e-2 relative, with 1e-3 of the rows' RMS as the floor
// for entries that cancel).  One line per tile in the format of the int32 sweep.
int sweep_group_scales(int M, int N, int K, int x_bits, int w_bits, bool is_signed, int group, bool fp6, const std::vector<int> &h_x,
                       const std::vector<int> &h_w, const uint32_t *d_xp, const uint32_t *d_xt, const uint32_t *d_wt,
                       const uint32_t *d_wf, size_t wp_bytes, size_t wf_bytes, size_t nbuf, int repeat, int warmup,
                       const std::string &only, hipStream_t stream)
{
    if ((group != 64 && group != 128) || K % group) {
        std::printf("Error, --group takes 64 or 128\n");
        return -1;
    }
    if (fp6 && (!d_wf || group != 128)) {
        std::printf("Error, --fp6 needs a bit pair that qualifies for FP6 records and groups of 128\n");
        return -1;
    }
    const int G = K / group;
    std::mt19937 rng(7);
    std::uniform_real_distribution<float> sd(0.001f, 0.011f);
    std::vector<float> h_ws((size_t)N * G), h_wz((size_t)N * G), h_xs(M);
    const int wlo = is_signed ? -(1 << (w_bits - 1)) : 0;
    for (auto &v : h_ws)
        v = sd(rng);
    for (auto &v : h_wz)
        v = (float)(wlo + (int)(rng() % (1u << w_bits)));
    for (auto &v : h_xs)
        v = sd(rng);
    std::vector<int> h_sums((size_t)M * G);
    for (int m = 0; m < M; ++m)
        for (int g = 0; g < G; ++g) {
            int sum = 0;
            for (int k = 0; k < group; ++k)
                sum += h_x[(size_t)m * K + (size_t)g * group + k];
            h_sums[(size_t)m * G + g] = sum;
        }
    // expected values of the sampled rows
    const int nrows = std::min(M, 8);
    std::vector<int> rows(nrows);
    for (int i = 0; i < nrows; ++i)
        rows[i] = (int)((long)i * (M - 1) / std::max(1, nrows - 1));
    std::vector<double> want((size_t)nrows * N);
    double sq = 0;
#pragma omp parallel for collapse(2) schedule(static) reduction(+ : sq)
    for (int i = 0; i < nrows; ++i)
        for (int n = 0; n < N; ++n) {
            const int *xr = &h_x[(size_t)rows[i] * K], *wr = &h_w[(size_t)n * K];
            double v = 0;
            for (int g = 0; g < G; ++g) {
                long acc = 0;
                for (int k = g * group; k < (g + 1) * group; ++k)
                    acc += (long)xr[k] * wr[k];
                v += (double)h_ws[(size_t)n * G + g] * ((double)acc - (double)h_wz[(size_t)n * G + g] * h_sums[(size_t)rows[i] * G + g]);
            }
            v *= h_xs[rows[i]];
            want[(size_t)i * N + n] = v;
            sq += v * v;
        }
    const double rms = std::sqrt(sq / ((double)nrows * N));

    float *d_ws_, *d_wz_, *d_xs_;
    int *d_sums;
    uint16_t *d_out; // fp16
    uint32_t *d_xf = nullptr;
    HIP_OK(hipMalloc(&d_ws_, h_ws.size() * 4));
    HIP_OK(hipMalloc(&d_wz_, h_wz.size() * 4));
    HIP_OK(hipMalloc(&d_xs_, h_xs.size() * 4));
    HIP_OK(hipMalloc(&d_sums, h_sums.size() * 4));
    HIP_OK(hipMalloc(&d_out, (size_t)M * N * 2));
    HIP_OK(hipMemcpy(d_ws_, h_ws.data(), h_ws.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_wz_, h_wz.data(), h_wz.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_xs_, h_xs.data(), h_xs.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_sums, h_sums.data(), h_sums.size() * 4, hipMemcpyHostToDevice));
    if (fp6) {
        HIP_OK(hipMalloc(&d_xf, abq_fp6_bytes(M, K)));
        if (abq_relayout_planes_fp6(d_xp, d_xf, M, K, x_bits, is_signed, stream) != ABQ_OK) {
            std::printf("abq_relayout_planes_fp6 failed (hip error %d)\n", abq_last_hip_error());
            return -1;
        }
    }
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    const int layout = fp6 ? ABQ_LAYOUT_FP6 : ABQ_LAYOUT_TILED;
    const double ops = 2.0 * M * N * K;
    std::vector<uint16_t> h_out((size_t)M * N);
    std::vector<std::string> seen;
    double best_tops = 0;
    std::string best;
    const int ncfg = abq_native_config_count(x_bits, w_bits, is_signed);
    for (int i = 0; i <= ncfg; ++i) {
        abq_tile_config cfg;
        const bool library_default = i == ncfg;
        if (!library_default) {
            if (abq_native_config_get(x_bits, w_bits, is_signed, i, &cfg) != ABQ_OK || cfg.nstage != (fp6 ? 5 : 4) || cfg.warp_k != 128)
                continue;
            char name[160];
            abq_format_kernel_name(&cfg, 0, name, sizeof name);
            if (!only.empty() && std::string(name).find(only) == std::string::npos)
                continue;
        }
        std::vector<abq_gemm_state> states(nbuf);
        bool ok = true;
        for (size_t b = 0; b < nbuf && ok; ++b) {
            const char *wbase = fp6 ? (const char *)d_wf + b * wf_bytes : (const char *)d_wt + b * wp_bytes;
            abq_status s = abq_gemm_init(library_default ? nullptr : &cfg, x_bits, w_bits, is_signed, fp6 ? d_xf : d_xt,
                                         (const uint32_t *)wbase, M, N, K, d_out, nullptr, 0, ABQ_OUT_F16_SCALED, &states[b]);
            if (s == ABQ_OK)
                s = abq_gemm_set_operand_layout(&states[b], layout, layout);
            if (s == ABQ_OK)
                s = abq_gemm_set_scales(&states[b], d_xs_, d_ws_, group);
            if (s == ABQ_OK)
                s = abq_gemm_set_zero_points(&states[b], nullptr, d_wz_, d_sums, nullptr);
            ok = s == ABQ_OK && states[b].init_success;
        }
        if (!ok)
            continue; // no group-scale build of this tile
        const abq_tile_config &c = states[0].cfg;
        char key[96];
        std::snprintf(key, sizeof key, "%d %d %d %d %d %d %zu", c.block_m, c.block_n, c.block_k, c.warp_m, c.warp_n, c.nstage, states[0].shared_mem_size);
        if (!library_default) {
            if (std::find(seen.begin(), seen.end(), key) != seen.end())
                continue; // tuples that resolve to the same group-scale kernel
            seen.push_back(key);
        }
        HIP_OK(hipMemsetAsync(d_out, 0xff, (size_t)M * N * 2, stream));
        int status = 0;
        if (abq_gemm_exec(&states[0], stream) != ABQ_OK || hipStreamSynchronize(stream) != hipSuccess)
            status = -1;
        if (status == 0) {
            HIP_OK(hipMemcpy(h_out.data(), d_out, (size_t)M * N * 2, hipMemcpyDeviceToHost));
            for (int r = 0; r < nrows && status == 0; ++r)
                for (int n = 0; n < N; ++n) {
                    const double got = half_bits_to_double(h_out[(size_t)rows[r] * N + n]), w = want[(size_t)r * N + n];
                    if (!(std::fabs(got - w) <= 1e-2 * std::fabs(w) + 1e-3 * rms)) {
                        status = -2;
                        break;
                    }
                }
        }
        float ms = 0;
        if (status != -1) { // a tile whose values failed the check is still timed, like in the int32 sweep
            for (int j = 0; j < warmup; ++j)
                abq_gemm_exec(&states[j % nbuf], stream);
            hipGraph_t g;
            hipGraphExec_t ge;
            HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
            for (int j = 0; j < repeat; ++j)
                abq_gemm_exec(&states[j % nbuf], stream);
            HIP_OK(hipStreamEndCapture(stream, &g));
            HIP_OK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
            warm_replays(ge, stream);
            HIP_OK(hipEventRecord(e0, stream));
            HIP_OK(hipGraphLaunch(ge, stream));
            HIP_OK(hipEventRecord(e1, stream));
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            HIP_OK(hipGraphExecDestroy(ge));
            HIP_OK(hipGraphDestroy(g));
        }
        const float us = ms * 1e3f / repeat;
        const double tops = status == 0 ? ops / (us * 1e-6) / 1e12 : 0;
        std::printf("gfx950 W%dA%d %s group %d%s %d %d %d %d %d %d %d %d %d %d lds %zu exec %f (us) %f TOPS | %s | %.1f%% MFMA%s\n", w_bits,
                    x_bits, is_signed ? "int" : "uint", group, fp6 ? " FP6" : "", c.block_m, c.block_n, c.block_k, c.warp_m, c.warp_n,
                    c.warp_k, c.mma_m, c.mma_n, c.mma_k, c.nstage, states[0].shared_mem_size, us, tops,
                    status == 0 ? "PASSED" : status == -1 ? "ERROR" : "FAILED", 100.0 * tops / 5000.0,
                    library_default ? " | library default" : "");
        if (status == 0 && !library_default && tops > best_tops) {
            best_tops = tops;
            char buf[128];
            std::snprintf(buf, sizeof buf, "%d, %d, %d, %d, %d, %d, %d, %d, %d, %d", c.block_m, c.block_n, c.block_k, c.warp_m, c.warp_n,
                          c.warp_k, c.mma_m, c.mma_n, c.mma_k, c.nstage);
            best = buf;
        }
        std::fflush(stdout);
    }
    std::printf("The best kernel config is %s with %f TOPS\n", best.c_str(), best_tops);
    (void)hipFree(d_ws_);
    (void)hipFree(d_wz_);
    (void)hipFree(d_xs_);
    (void)hipFree(d_sums);
    (void)hipFree(d_out);
    if (d_xf)
        (void)hipFree(d_xf);
    return 0;
}

} // namespace

int main(int argc, char **argv)
{
    if (argc < 7) {
        std::printf("Usage: ./test_any_mma M N K X_BITS W_BITS SIGNED [--repeat R] [--warmup W] [--rotate-mib MiB] [--stream] [--only SUBSTR] [--seed S] [--read-floor] [--zero-operands] [--mfma-ceiling] [--group 64|128 [--fp6]]\n");
        return -1;
    }
    const int M = std::atoi(argv[1]), N = std::atoi(argv[2]), K = std::atoi(argv[3]);
    const int x_bits = std::atoi(argv[4]), w_bits = std::atoi(argv[5]);
    const bool is_signed = std::atoi(argv[6]) == 1;
    int repeat = 1000, warmup = 10, rotate_mib = 512;
    bool use_graph = true, read_floor = false, group_fp6 = false, mfma_ceiling = false, zero_operands = false;
    int group = 0; // --group: sweep the tiles of the kernels with group scales and zero points (fp16 out) instead
    unsigned long seed = 0;
    std::string only, tuning_in, tuning_out;
    for (int i = 7; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--stream"))
            use_graph = false;
        else if (!std::strcmp(argv[i], "--read-floor"))
            read_floor = true;
        else if (!std::strcmp(argv[i], "--fp6"))
            group_fp6 = true;
        else if (!std::strcmp(argv[i], "--zero-operands"))
            zero_operands = true;
        else if (!std::strcmp(argv[i], "--mfma-ceiling"))
            mfma_ceiling = true;
        else if (i + 1 < argc && !std::strcmp(argv[i], "--group"))
            group = std::atoi(argv[++i]);
        else if (i + 1 < argc && !std::strcmp(argv[i], "--repeat"))
            repeat = std::atoi(argv[++i]);
        else if (i + 1 < argc && !std::strcmp(argv[i], "--warmup"))
            warmup = std::atoi(argv[++i]);
        else if (i + 1 < argc && !std::strcmp(argv[i], "--rotate-mib"))
            rotate_mib = std::atoi(argv[++i]);
        else if (i + 1 < argc && !std::strcmp(argv[i], "--only"))
            only = argv[++i];
        else if (i + 1 < argc && !std::strcmp(argv[i], "--tuning"))
            tuning_in = argv[++i];
        else if (i + 1 < argc && !std::strcmp(argv[i], "--tuning-out"))
            tuning_out = argv[++i];
        else if (!std::strcmp(argv[i], "--no-builtin-tuning"))
            abq_tuning_enable_builtin(0);
        else if (i + 1 < argc && !std::strcmp(argv[i], "--seed"))
            seed = std::strtoul(argv[++i], nullptr, 10);
    }
    if (K < 128 || K % 128 != 0) { // engine/test_any_mma.cu:99
        std::printf("Error, k must >= 128 and k %% 128 == 0!");
        return -1;
    }
    if (!tuning_in.empty()) {
        int taken = 0;
        if (abq_tuning_load(tuning_in.c_str(), &taken) != ABQ_OK) {
            std::printf("Error, cannot read the tuning table %s\n", tuning_in.c_str());
            return -1;
        }
        std::printf("tuning table %s: %d entries\n", tuning_in.c_str(), taken);
    }

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    if (mfma_ceiling)
        return matrix_core_ceiling(stream);

    // ---- host operands: uniform over the full range of the bit width
    std::mt19937_64 rng(seed);
    auto fill = [&](std::vector<int> &v, int bits) {
        const int lo = is_signed ? -(1 << (bits - 1)) : 0;
        const int span = 1 << bits;
        for (auto &e : v)
            e = zero_operands ? 0 : lo + (int)(rng() % (unsigned long)span);
    };
    std::vector<int> h_x((size_t)M * K), h_w((size_t)N * K);
    fill(h_x, x_bits);
    fill(h_w, w_bits);

    const size_t KW = K / 32;
    const size_t xp_words = (size_t)x_bits * M * KW, wp_words = (size_t)w_bits * N * KW;
    const size_t wp_bytes = wp_words * 4;
    size_t nbuf = std::max<size_t>(1, ((size_t)rotate_mib << 20) / wp_bytes);
    nbuf = std::min<size_t>(nbuf, 4096);

    int *d_x, *d_w, *d_out;
    uint32_t *d_xp, *d_wp;
    HIP_OK(hipMalloc(&d_x, h_x.size() * 4));
    HIP_OK(hipMalloc(&d_w, h_w.size() * 4));
    HIP_OK(hipMalloc(&d_xp, xp_words * 4));
    HIP_OK(hipMalloc(&d_wp, wp_bytes * nbuf));
    HIP_OK(hipMalloc(&d_out, (size_t)M * N * 4));
    HIP_OK(hipMemcpy(d_x, h_x.data(), h_x.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_w, h_w.data(), h_w.size() * 4, hipMemcpyHostToDevice));

    if (abq_pack_i32(d_w, d_wp, N, K, w_bits, stream) != ABQ_OK || abq_pack_i32(d_x, d_xp, M, K, x_bits, stream) != ABQ_OK) {
        std::printf("launch_pack failed (hip error %d)\n", abq_last_hip_error());
        return -1;
    }
    HIP_OK(hipStreamSynchronize(stream));
    for (size_t b = 1; b < nbuf; ++b)
        HIP_OK(hipMemcpyAsync((char *)d_wp + b * wp_bytes, d_wp, wp_bytes, hipMemcpyDeviceToDevice, stream));
    HIP_OK(hipStreamSynchronize(stream));

    // Weights for the kernels on the K-tiled layout are prepared once, like the packing itself;
    // activations stay in the reference layout and are converted inside every exec call.
    uint32_t *d_wt;
    char *d_ws;
    HIP_OK(hipMalloc(&d_wt, wp_bytes * nbuf));
    // (+ the activations' row sums, which exec takes for unsigned pairs with 8-bit weights when the activations arrive as planes)
    const size_t ws_bytes = std::max(abq_planes_bytes(M, K, abq_padded_bits(x_bits)), abq_fp6_bytes(M, K)) + (size_t)M * 4 + 1024;
    HIP_OK(hipMalloc(&d_ws, ws_bytes));
    if (abq_relayout_planes(d_wp, d_wt, N, K, w_bits, stream) != ABQ_OK) {
        std::printf("abq_relayout_planes failed (hip error %d)\n", abq_last_hip_error());
        return -1;
    }
    HIP_OK(hipStreamSynchronize(stream));
    for (size_t b = 1; b < nbuf; ++b)
        HIP_OK(hipMemcpyAsync((char *)d_wt + b * wp_bytes, d_wt, wp_bytes, hipMemcpyDeviceToDevice, stream));
    HIP_OK(hipStreamSynchronize(stream));

    // the decode kernel on K-tiled operands takes the activations in that layout too
    uint32_t *d_xt;
    HIP_OK(hipMalloc(&d_xt, xp_words * 4));
    if (abq_relayout_planes(d_xp, d_xt, M, K, x_bits, stream) != ABQ_OK) {
        std::printf("abq_relayout_planes failed (hip error %d)\n", abq_last_hip_error());
        return -1;
    }
    HIP_OK(hipStreamSynchronize(stream));

    // The FP6 kernels (NSTAGE 5) read their own record format: 96 bytes per row and K tile.
    const bool fp6_ok = abq_fp6_eligible(x_bits, w_bits, is_signed, K) != 0;
    const size_t wf_bytes = abq_fp6_bytes(N, K);
    uint32_t *d_wf = nullptr;
    if (fp6_ok) {
        HIP_OK(hipMalloc(&d_wf, wf_bytes * nbuf));
        if (abq_relayout_planes_fp6(d_wp, d_wf, N, K, w_bits, is_signed, stream) != ABQ_OK) {
            std::printf("abq_relayout_planes_fp6 failed (hip error %d)\n", abq_last_hip_error());
            return -1;
        }
        HIP_OK(hipStreamSynchronize(stream));
        for (size_t b = 1; b < nbuf; ++b)
            HIP_OK(hipMemcpyAsync((char *)d_wf + b * wf_bytes, d_wf, wf_bytes, hipMemcpyDeviceToDevice, stream));
        HIP_OK(hipStreamSynchronize(stream));
    }

    // Decode-sized M, prepared operands.  Weights of several fields (3, 5, 6, 7 bits) are read by the decode kernel as
    // the records above; activations of such widths come as padded records (abq_relayout_planes_padded: the next width
    // of 2, 4 or 8 bits), and unsigned 8-bit codes bring their row sums (abq_row_sums).  A second "prepared operands"
    // line times the same pairs with the weights padded as well (the padded pair's kernel).  Above 16 rows the padded
// weights get a line too: the padded pair's prefill kernel, the activations arriving as planes of their own width.
    const int xq = abq_padded_bits(x_bits), wq = abq_padded_bits(w_bits);
    const bool padded = xq != x_bits || wq != w_bits;
    const bool with_sums = !is_signed && (x_bits == 8 || w_bits == 8);
    const size_t wpad_bytes = abq_planes_bytes(N, K, wq);
    size_t nbuf_pad = std::min<size_t>(4096, std::max<size_t>(1, ((size_t)rotate_mib << 20) / wpad_bytes));
    uint32_t *d_xpad = nullptr, *d_wpad = nullptr;
    int *d_xsum = nullptr, *d_wsum = nullptr;
    if (with_sums) { // the weights' row sums belong to their preparation, whatever M is
        HIP_OK(hipMalloc(&d_xsum, (size_t)M * 4));
        HIP_OK(hipMalloc(&d_wsum, (size_t)N * 4));
        if (abq_row_sums(d_xp, M, K, x_bits, d_xsum, stream) != ABQ_OK || abq_row_sums(d_wp, N, K, w_bits, d_wsum, stream) != ABQ_OK) {
            std::printf("abq_row_sums failed (hip error %d)\n", abq_last_hip_error());
            return -1;
        }
    }
    // (above 16 rows only where the padded pair's weights are K-tiled records as well)
    const bool padded_prefill = M > 16 && padded && !group && abq_preferred_weight_layout(xq, wq, is_signed, M, N, K, 0) == ABQ_LAYOUT_TILED;
    const bool want_wpad = M <= 16 ? (padded || with_sums) : padded_prefill;
    if (want_wpad || xq != x_bits) { // (activations of several fields: what the NSTAGE 6 tiles read at any M)
        HIP_OK(hipMalloc(&d_xpad, abq_planes_bytes(M, K, xq)));
        if (abq_relayout_planes_padded(d_xp, d_xpad, M, K, x_bits, is_signed, stream) != ABQ_OK) {
            std::printf("preparing padded records failed (hip error %d)\n", abq_last_hip_error());
            return -1;
        }
        HIP_OK(hipStreamSynchronize(stream));
    }
    if (want_wpad) {
        HIP_OK(hipMalloc(&d_wpad, wpad_bytes * nbuf_pad));
        if (abq_relayout_planes_padded(d_wp, d_wpad, N, K, w_bits, is_signed, stream) != ABQ_OK) {
            std::printf("preparing padded records failed (hip error %d)\n", abq_last_hip_error());
            return -1;
        }
        HIP_OK(hipStreamSynchronize(stream));
        for (size_t b = 1; b < nbuf_pad; ++b)
            HIP_OK(hipMemcpyAsync((char *)d_wpad + b * wpad_bytes, d_wpad, wpad_bytes, hipMemcpyDeviceToDevice, stream));
        HIP_OK(hipStreamSynchronize(stream));
    }

    if (group)
        return sweep_group_scales(M, N, K, x_bits, w_bits, is_signed, group, group_fp6, h_x, h_w, d_xp, d_xt, d_wt, d_wf, wp_bytes,
                                  wf_bytes, nbuf, repeat, warmup, only, stream);

    std::vector<uint32_t> h_xp(xp_words), h_wp(wp_words);
    HIP_OK(hipMemcpy(h_xp.data(), d_xp, xp_words * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(h_wp.data(), d_wp, wp_words * 4, hipMemcpyDeviceToHost));
    std::vector<int> h_ref((size_t)M * N), h_out((size_t)M * N);
    expected_result(h_wp, h_xp, h_ref, M, N, K, w_bits, x_bits, is_signed);

    // ---- activation packing time (reported separately, test_mma.h:141-152)
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    float pack_us = 0;
    {
        for (int i = 0; i < warmup; ++i)
            abq_pack_i32(d_x, d_xp, M, K, x_bits, stream);
        HIP_OK(hipEventRecord(e0, stream));
        const int reps = std::max(10, repeat / 10);
        for (int i = 0; i < reps; ++i)
            abq_pack_i32(d_x, d_xp, M, K, x_bits, stream);
        HIP_OK(hipEventRecord(e1, stream));
        HIP_OK(hipStreamSynchronize(stream));
        float ms;
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        pack_us = ms * 1e3f / reps;
    }

    const double ops = 2.0 * M * N * K;
    const double alg_bytes = (double)w_bits * N * K / 8 + (double)x_bits * M * K / 8 + 4.0 * M * N;
    char config_str[32];
    std::snprintf(config_str, sizeof config_str, "W%dA%d %s", w_bits, x_bits, is_signed ? "int" : "uint");

    // the layout a loader would hold the weights in for this shape (the library's own choice above 16 rows)
    const int preferred = abq_preferred_weight_layout(x_bits, w_bits, is_signed, M, N, K, 0);
    // ... and when the table's tile for the shape is the decode kernel of prepared operands, the activations come
    // K-tiled too, as the quantising kernel writes them (what that tile's own line of the sweep is timed on)
    abq_tile_config tuned;
    const bool tuned_decode = M > 16 && abq_tuning_lookup(x_bits, w_bits, is_signed, M, N, K, 0, 0, &tuned, nullptr) == ABQ_OK && tuned.nstage == 6;
    const bool x_fields = xq != x_bits; // activations the decode kernel reads as padded records
    auto run_one = [&](const abq_tile_config *cfg, Timing &t, abq_gemm_state &st0, bool prepared = false, bool pad_weights = false) {
        std::vector<abq_gemm_state> states(nbuf);
        // tiled tiles (NSTAGE 4) run on prepared weights, NSTAGE 6 and the `prepared` default on prepared weights and
        // activations, the FP6 tiles on FP6 records; the library's own choice for M > 16 on the preferred layout
        // (the default with the weights as padded records: the padded pair's kernel)
        const bool via_padded = !cfg && pad_weights && d_wpad != nullptr;
        const bool both = prepared || (cfg ? cfg->nstage == 6 : (tuned_decode && !via_padded));
        const bool fp6 = cfg ? cfg->nstage == 5 : (!prepared && !via_padded && M > 16 && preferred == ABQ_LAYOUT_FP6 && fp6_ok);
        const bool tiled = both || via_padded || (cfg ? cfg->nstage == 4 : (M > 16 && !fp6 && preferred != ABQ_LAYOUT_PLANES));
        if (fp6 && !fp6_ok) {
            t.status = -1;
            return;
        }
        if (via_padded)
            states.resize(nbuf_pad);
        if (both && x_fields && !d_xpad) { // more than 16 rows: no padded activations were made
            t.status = -1;
            return;
        }
        for (size_t b = 0; b < states.size(); ++b) {
            const char *wbase = via_padded ? (const char *)d_wpad + b * wpad_bytes
                                : fp6      ? (const char *)d_wf + b * wf_bytes
                                           : (tiled ? (const char *)d_wt : (const char *)d_wp) + b * wp_bytes;
            abq_status s = abq_gemm_init(cfg, via_padded ? xq : x_bits, via_padded ? wq : w_bits, is_signed,
                                         !both ? d_xp : via_padded ? d_xpad : (x_fields ? d_xpad : d_xt), (const uint32_t *)wbase,
                                         M, N, K, d_out, nullptr, 0, ABQ_OUT_I32, &states[b]);
            if (s == ABQ_OK && via_padded && padded)
                s = abq_gemm_set_value_bits(&states[b], x_bits, w_bits);
            if (s == ABQ_OK && both && !via_padded && x_fields)
                s = abq_gemm_set_padded_activations(&states[b], 1);
            // unsigned 8-bit codes: the weights' row sums come with the prepared weights; the activations' with prepared
            // activations, else exec takes them from the planes into the workspace
            if (s == ABQ_OK && (both || tiled) && with_sums)
                s = abq_gemm_set_row_sums(&states[b], both ? d_xsum : nullptr, d_wsum);
            if (s == ABQ_OK && tiled)
                s = abq_gemm_set_operand_layout(&states[b], both ? ABQ_LAYOUT_TILED : ABQ_LAYOUT_PLANES, ABQ_LAYOUT_TILED);
            if (s == ABQ_OK && fp6)
                s = abq_gemm_set_operand_layout(&states[b], ABQ_LAYOUT_PLANES, ABQ_LAYOUT_FP6);
            if (s == ABQ_OK && (tiled || fp6))
                s = abq_gemm_set_workspace(&states[b], d_ws, ws_bytes);
            if (s != ABQ_OK || !states[b].init_success) {
                t.status = -1;
                return;
            }
        }
        st0 = states[0];
        HIP_OK(hipMemsetAsync(d_out, 0xff, (size_t)M * N * 4, stream));
        if (abq_gemm_exec(&states[0], stream) != ABQ_OK || hipStreamSynchronize(stream) != hipSuccess) {
            t.status = -1;
            return;
        }
        HIP_OK(hipMemcpy(h_out.data(), d_out, (size_t)M * N * 4, hipMemcpyDeviceToHost));
        t.status = std::memcmp(h_out.data(), h_ref.data(), (size_t)M * N * 4) == 0 ? 0 : -2;
        for (int i = 0; i < warmup; ++i)
            abq_gemm_exec(&states[i % states.size()], stream);
        HIP_OK(hipStreamSynchronize(stream));
        float ms = 0;
        if (use_graph) {
            hipGraph_t g;
            hipGraphExec_t ge;
            HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
            for (int i = 0; i < repeat; ++i)
                abq_gemm_exec(&states[i % states.size()], stream);
            HIP_OK(hipStreamEndCapture(stream, &g));
            HIP_OK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
            warm_replays(ge, stream);
            HIP_OK(hipEventRecord(e0, stream));
            HIP_OK(hipGraphLaunch(ge, stream));
            HIP_OK(hipEventRecord(e1, stream));
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            HIP_OK(hipGraphExecDestroy(ge));
            HIP_OK(hipGraphDestroy(g));
        } else {
            HIP_OK(hipEventRecord(e0, stream));
            for (int i = 0; i < repeat; ++i)
                abq_gemm_exec(&states[i % states.size()], stream);
            HIP_OK(hipEventRecord(e1, stream));
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        }
        t.exec_us = ms * 1e3f / repeat;
        t.pack_us = pack_us;
    };

    double best_tops = 0;
    std::string best;
    // the fastest tile of each operand layout (planes, K-tiled, FP6), for --tuning-out
    double layout_tops[3] = { 0, 0, 0 };
    abq_tile_config layout_best[3];
    const int ncfg = abq_native_config_count(x_bits, w_bits, is_signed);
    // + the library's choice (+ its choice on prepared operands (+ the same with the weights padded as well))
    const int nlines = ncfg + (M <= 16 ? (padded && wq != w_bits ? 3 : 2) : (padded_prefill ? 2 : 1));
    for (int i = 0; i < nlines; ++i) {
        abq_tile_config cfg;
        const bool library_default = i >= ncfg;
        const bool prepared = M <= 16 && i >= ncfg + 1, pad_weights = i == ncfg + (M <= 16 ? 2 : 1);
        if (!library_default && abq_native_config_get(x_bits, w_bits, is_signed, i, &cfg) != ABQ_OK)
            continue;
        char name[160] = "library default";
        const char *how = pad_weights ? " (padded records)" : (with_sums && d_wpad) ? " (with row sums)" : "";
        if (prepared)
            std::snprintf(name, sizeof name, "library default, prepared operands%s", how);
        else if (pad_weights)
            std::snprintf(name, sizeof name, "library default (padded records)");
        if (!library_default)
            abq_format_kernel_name(&cfg, 0, name, sizeof name);
        if (!only.empty() && std::string(name).find(only) == std::string::npos)
            continue;
        Timing t;
        abq_gemm_state st;
        std::memset(&st, 0, sizeof st);
        run_one(library_default ? nullptr : &cfg, t, st, prepared, pad_weights);
        const abq_tile_config &c = st.cfg;
        const double tops = t.status == 0 ? ops / (t.exec_us * 1e-6) / 1e12 : 0;
        std::printf("gfx950 %s %d %d %d %d %d %d %d %d %d %d ", config_str, c.block_m, c.block_n, c.block_k, c.warp_m,
                    c.warp_n, c.warp_k, c.mma_m, c.mma_n, c.mma_k, c.nstage);
        std::printf("packing %f (us) exec %f (us) %f TOPS | %f B-TOPS | %s | %.1f%% HBM %.1f%% MFMA%s\n", t.pack_us,
                    t.exec_us, tops, tops * x_bits * w_bits, t.status == 0 ? "PASSED" : t.status == -1 ? "ERROR" : "FAILED",
                    t.status == 0 ? 100.0 * alg_bytes / (t.exec_us * 1e-6) / 8e12 : 0.0, 100.0 * tops / 5000.0,
                    prepared ? (pad_weights ? " | library default, prepared operands (padded records)"
                                : (with_sums && d_wpad) ? " | library default, prepared operands (with row sums)"
                                                        : " | library default, prepared operands")
                    : pad_weights   ? " | library default (padded records)"
                    : library_default ? " | library default" : "");
        if (t.status == 0 && !library_default && tops > best_tops) {
            best_tops = tops;
            char buf[128];
            std::snprintf(buf, sizeof buf, "%d, %d, %d, %d, %d, %d, %d, %d, %d, %d", c.block_m, c.block_n, c.block_k, c.warp_m,
                          c.warp_n, c.warp_k, c.mma_m, c.mma_n, c.mma_k, c.nstage);
            best = buf;
        }
        if (t.status == 0 && !library_default) {
            const int layout = c.nstage == 5 ? ABQ_LAYOUT_FP6 : (c.nstage == 4 || c.nstage == 6) ? ABQ_LAYOUT_TILED : ABQ_LAYOUT_PLANES;
            if (tops > layout_tops[layout]) {
                layout_tops[layout] = tops;
                layout_best[layout] = c;
            }
        }
        std::fflush(stdout);
    }
    std::printf("The best kernel config is %s with %f TOPS\n", best.c_str(), best_tops);
    if (!tuning_out.empty() && only.empty()) {
        // one line per operand layout that has a passing tile: what abq_tuning_load and the compiled-in table read
        FILE *f = std::fopen(tuning_out.c_str(), "a");
        if (!f) {
            std::printf("Error, cannot append to %s\n", tuning_out.c_str());
            return -1;
        }
        for (int layout = 0; layout < 3; ++layout) {
            if (layout_tops[layout] <= 0)
                continue;
            char name[160];
            abq_format_kernel_name(&layout_best[layout], 0, name, sizeof name);
            std::fprintf(f, "%s %d %d %d 0 %.1f\n", name, M, N, K, layout_tops[layout]);
        }
        std::fclose(f);
    }

    if (read_floor) {
        auto time_probe = [&](int kind) {
            auto body = [&](int count) {
                for (int i = 0; i < count; ++i)
                    abq_probe_launch(kind, (const char *)d_wp + (size_t)(i % nbuf) * wp_bytes, wp_bytes, stream);
            };
            body(warmup);
            HIP_OK(hipStreamSynchronize(stream));
            float ms = 0;
            hipGraph_t g;
            hipGraphExec_t ge;
            if (use_graph) {
                HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
                body(repeat);
                HIP_OK(hipStreamEndCapture(stream, &g));
                HIP_OK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
                warm_replays(ge, stream);
            }
            HIP_OK(hipEventRecord(e0, stream));
            if (use_graph)
                HIP_OK(hipGraphLaunch(ge, stream));
            else
                body(repeat);
            HIP_OK(hipEventRecord(e1, stream));
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            if (use_graph) {
                HIP_OK(hipGraphExecDestroy(ge));
                HIP_OK(hipGraphDestroy(g));
            }
            return ms * 1e3f / repeat;
        };
        const float empty_us = time_probe(ABQ_PROBE_EMPTY), read_us = time_probe(ABQ_PROBE_READ);
        std::printf("floor: empty kernel %f (us) | read of the %zu packed weight bytes, 16-byte loads, no compute %f (us) = %.1f%% HBM\n",
                    empty_us, wp_bytes, read_us, 100.0 * (double)wp_bytes / (read_us * 1e-6) / 8e12);
    }

    (void)hipFree(d_x);
    (void)hipFree(d_w);
    (void)hipFree(d_xp);
    (void)hipFree(d_wp);
    (void)hipFree(d_out);
    (void)hipFree(d_wt);
    (void)hipFree(d_xt);
    if (d_wf)
        (void)hipFree(d_wf);
    (void)hipFree(d_ws);
    (void)hipStreamDestroy(stream);
    return 0;
}
