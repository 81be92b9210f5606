// Table of measured best tiles: the result of the autotune sweep, consulted before the fitted rules.
//
// In the reference the sweep's "The best kernel config is ..." line (engine/test/test_mma/test_mma.h:21-45,
// test_mma_w2a8.cu:700) ends up hard-coded in the FT wrapper
// (fastertransformer/src/fastertransformer/kernels/abqgemm/abq_gemm_wrapper.cu:105-124).  Here the harness
// (engine/test_any_mma --tuning-out) appends its best lines to a text file; the file shipped with the library is
// compiled in (abq_tuning_default.inc, made from engine/tuning_mi355x.txt by the Makefile), more can be loaded at
// run time, and abq_gemm_init(cfg = NULL) and the calls that declare layouts, scales and workspace look a shape up
// here first and fall back to their rules.
//
// One line per entry, '#' starts a comment:
//     <kernel name> <M> <N> <K> <group size> <TOPS>
// The kernel name carries bit widths, signedness and the tile tuple (abq_parse_kernel_name); the tuple says which
// operand layout the tile runs on (NSTAGE 5: FP6 records; NSTAGE 4 and 6: K-tiled; else planes).  An entry serves
// the M of its bucket (1, 2, 3-4, 5-8, 9-16, 17-32, 33-64, ...) on exactly its N, K and group size.  A file may hold
// several entries per shape, e.g. the best tile of each layout: a lookup takes the fastest among those the caller
// can run.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>

#include "abq_gemm.h"
#include "abq_tuning.h"

namespace abq {

namespace {

const char *const kBuiltin[] = {
#include "abq_tuning_default.inc"
    nullptr
};

std::mutex g_mutex;
std::vector<TunedTile> g_loaded;   // abq_tuning_load / abq_tuning_add, in order of arrival
std::vector<TunedTile> g_builtin;  // parsed on first use
bool g_builtin_parsed = false;
bool g_builtin_enabled = true;

int m_bucket(int M)
{
    if (M <= 2)
        return M <= 1 ? 0 : 1;
    int b = 2, top = 4;
    while (M > top) {
        top *= 2;
        ++b;
    }
    return b;
}

// "<name> M N K group tops"; false on a malformed line
bool parse_line(const char *line, TunedTile *out)
{
    char name[192];
    int M, N, K, group;
    float tops = 0.f;
    const int n = sscanf(line, "%191s %d %d %d %d %f", name, &M, &N, &K, &group, &tops);
    if (n < 5)
        return false;
    abq_tile_config cfg;
    if (abq_parse_kernel_name(name, &cfg, nullptr) != ABQ_OK)
        return false;
    if (M <= 0 || N <= 0 || K < 128 || K % 128 != 0 || (group != 0 && group != 64 && group != 128))
        return false;
    *out = TunedTile{ cfg, M, N, K, group, tops };
    return true;
}

void parse_builtin_locked()
{
    if (g_builtin_parsed)
        return;
    g_builtin_parsed = true;
    for (int i = 0; kBuiltin[i]; ++i) {
        TunedTile t;
        if (parse_line(kBuiltin[i], &t))
            g_builtin.push_back(t);
    }
}

const TunedTile *best_of(const std::vector<TunedTile> &table, int x_bits, int w_bits, int is_signed, int M, int N, int K, int group,
                         int layout_mask)
{
    const TunedTile *best = nullptr;
    const int bucket = m_bucket(M);
    for (const TunedTile &t : table) {
        if (t.cfg.x_bits != x_bits || t.cfg.w_bits != w_bits || (t.cfg.is_signed != 0) != (is_signed != 0) || t.N != N || t.K != K ||
            t.group_size != group || m_bucket(t.M) != bucket)
            continue;
        if (!(layout_mask & (1 << tile_operand_layout(t.cfg))))
            continue;
        // among the entries of a table the fastest; at equal figures the later line
        if (!best || t.tops >= best->tops)
            best = &t;
    }
    return best;
}

} // namespace

int tile_operand_layout(const abq_tile_config &c)
{
    if (c.mma_m == 32 && c.mma_n == 32 && c.mma_k == 64)
        return ABQ_LAYOUT_FP6;
    if ((c.mma_m == 32 && c.mma_k == 32 && c.nstage == 4) || (c.mma_m == 16 && c.mma_k == 64 && c.nstage == 6))
        return ABQ_LAYOUT_TILED;
    return ABQ_LAYOUT_PLANES;
}

bool tuning_find(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group, int layout_mask, TunedTile *out)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    const TunedTile *t = best_of(g_loaded, x_bits, w_bits, is_signed, M, N, K, group, layout_mask);
    if (!t && g_builtin_enabled) {
        parse_builtin_locked();
        t = best_of(g_builtin, x_bits, w_bits, is_signed, M, N, K, group, layout_mask);
    }
    if (!t)
        return false;
    *out = *t;
    return true;
}

} // namespace abq

using namespace abq;

extern "C" {

abq_status abq_tuning_add(const abq_tile_config *cfg, int M, int N, int K, int group_size, float tops)
{
    if (!cfg || M <= 0 || N <= 0)
        return ABQ_ERR_INVALID_ARG;
    if (K < 128 || K % 128 != 0)
        return ABQ_ERR_BAD_K;
    if (group_size != 0 && group_size != 64 && group_size != 128)
        return ABQ_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_mutex);
    g_loaded.push_back(TunedTile{ *cfg, M, N, K, group_size, tops });
    return ABQ_OK;
}

abq_status abq_tuning_load(const char *path, int *entries)
{
    if (entries)
        *entries = 0;
    if (!path)
        return ABQ_ERR_INVALID_ARG;
    FILE *f = fopen(path, "r");
    if (!f)
        return ABQ_ERR_INVALID_ARG;
    std::vector<TunedTile> fresh;
    char line[512];
    bool ok = true;
    while (ok && fgets(line, sizeof line, f)) {
        const char *p = line;
        while (*p == ' ' || *p == '\t')
            ++p;
        if (*p == '#' || *p == '\n' || *p == '\r' || *p == '\0')
            continue;
        TunedTile t;
        ok = parse_line(p, &t);
        if (ok)
            fresh.push_back(t);
    }
    fclose(f);
    if (!ok)
        return ABQ_ERR_INVALID_ARG; // a malformed line: nothing of the file is taken
    std::lock_guard<std::mutex> lock(g_mutex);
    g_loaded.insert(g_loaded.end(), fresh.begin(), fresh.end());
    if (entries)
        *entries = (int)fresh.size();
    return ABQ_OK;
}

void abq_tuning_clear(void)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    g_loaded.clear();
}

void abq_tuning_enable_builtin(int on)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    g_builtin_enabled = on != 0;
}

abq_status abq_tuning_lookup(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size, int layout_mask,
                             abq_tile_config *cfg, float *tops)
{
    if (!cfg)
        return ABQ_ERR_INVALID_ARG;
    TunedTile t;
    if (!tuning_find(x_bits, w_bits, is_signed, M, N, K, group_size, layout_mask ? layout_mask : 7, &t))
        return ABQ_ERR_UNSUPPORTED;
    *cfg = t.cfg;
    if (tops)
        *tops = t.tops;
    return ABQ_OK;
}

int abq_preferred_weight_layout(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size)
{
    // (signed 5-bit weights under activations that qualify too: the padded pair would be W8A8, and twice the int8 rate
    // beats its staged kernel: W5A5 128 x 5120 x 13824 575 against 517 TOPS; abq_preferred_weight_records says the same)
    if (M > 16 && is_signed && w_bits == 5 && abq_fp6_eligible(x_bits, w_bits, is_signed, K) && (group_size == 0 || group_size == 128))
        return ABQ_LAYOUT_FP6;
    if (activations_run_padded(x_bits, w_bits, is_signed, M, group_size))
        return ABQ_LAYOUT_TILED; // (whatever was measured on the pair's own kernels: the padded pair's run on these)
    TunedTile t;
    if (tuning_find(x_bits, w_bits, is_signed, M, N, K, group_size, 7, &t))
        return tile_operand_layout(t.cfg);
    // no measurement: FP6 records for the pairs that qualify once the GEMM is prefill-sized (the FP6 matrix cores run
    // at twice the int8 rate and nothing is unpacked), K-tiled records otherwise (every decode and prefill kernel
    // that is not the FP6 one runs fastest on them).  Up to 256 rows the int8 route's small tiles, whose waves split
    // K, are level or ahead (W4A4 / W2A2, activations converted in the call, int8 / FP6 us: 128 x 4096 x 4096 12.0 /
    // 13.9, 128 x 4096 x 11008 20.4 / 26.0, 256 x 4096 x 4096 13.1 / 14.4, 256 x 11008 x 4096 22.8 / 23.1; 384 x 11008 x 4096
    // 31.5 / 27.2, 512 x 4096 x 4096 with prepared activations 12.5 / 10.9).
    // Weights of at most 2 bits are 32 bytes per row and K tile on the int8 route against 96 as FP6 records: level only
    // from 2048 rows (W2A2 768 x 4096 x 4096 20.1 / 26.2, 1024 x 11008 x 4096 42.6 / 51.9, 2048 x 4096 x 4096 33.0 / 28.9,
    // 2048 x 11008 x 4096 72.8 / 75.7).
    if (M > (w_bits <= 2 ? 1024 : 256) && abq_fp6_eligible(x_bits, w_bits, is_signed, K) && (group_size == 0 || group_size == 128))
        return ABQ_LAYOUT_FP6;
    return ABQ_LAYOUT_TILED;
}

int abq_preferred_weight_records(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size, int *record_bits)
{
    const int wq = abq_padded_bits(w_bits);
    int bits = w_bits, layout;
    if (wq == w_bits || wq == 0) {
        layout = abq_preferred_weight_layout(x_bits, w_bits, is_signed, M, N, K, group_size);
    } else if (M > 16 && is_signed && w_bits == 5 && abq_fp6_eligible(x_bits, w_bits, is_signed, K) && (group_size == 0 || group_size == 128)) {
        layout = ABQ_LAYOUT_FP6; // twice the int8 rate beats the 8-bit records' staged kernel
    } else {
        // the padded pair's answer; FP6 records hold the codes themselves, whatever width they were declared with
        layout = abq_preferred_weight_layout(abq_padded_bits(x_bits), wq, is_signed, M, N, K, group_size);
        if (layout == ABQ_LAYOUT_FP6 && !abq_fp6_eligible(x_bits, w_bits, is_signed, K))
            layout = ABQ_LAYOUT_TILED;
        if (layout != ABQ_LAYOUT_FP6) {
            layout = ABQ_LAYOUT_TILED;
            bits = wq;
        }
    }
    if (record_bits)
        *record_bits = bits;
    return layout;
}

} // extern "C"
