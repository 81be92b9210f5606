// Host side of the C ABI declared in include/abq_gemm.h: argument checking, the kernel
// registry (tile tuple -> instantiation), the default strategy choice and the launches.
// No entry point allocates device or host memory.
#include "abq_gemm.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "abq_kernels.h"
#include "abq_tuning.h"

namespace abq {

hipError_t launch_pack_i32(const int32_t *, uint32_t *, int, int, int, hipStream_t);
hipError_t launch_pack_f16(const void *, const float *, uint32_t *, int, int, int, hipStream_t);
hipError_t launch_pack_f16_tiled(const void *, const float *, uint32_t *, int, int, int, hipStream_t);
hipError_t launch_pack_f16_fp6(const void *, const float *, uint32_t *, int, int, int, int, hipStream_t);
hipError_t launch_pack_u4(const uint32_t *, uint32_t *, int, int, int, hipStream_t);
hipError_t launch_relayout_planes(const uint32_t *, uint32_t *, int, int, int, hipStream_t);
hipError_t launch_relayout_planes_padded(const uint32_t *, uint32_t *, int, int, int, int, int, hipStream_t, int *row_sums = nullptr);
hipError_t launch_relayout_planes_folded(const uint32_t *, const float *, int, uint32_t *, int, int, int, int, int, int *, hipStream_t);
hipError_t launch_relayout_planes_fp6(const uint32_t *, uint32_t *, int, int, int, int, hipStream_t, const float *zero = nullptr,
                                      int group_size = 0, int *flag = nullptr);
hipError_t launch_row_sums(const uint32_t *, int *, int, int, int, hipStream_t);
const KernelEntry *fp6_entries(int *count);
const KernelEntry *fp6_grouped_entries(int *count);
hipError_t launch_quant_pack_rows(const void *, uint32_t *, float *, float *, int *, int, int, int, int, int, int,
                                  hipStream_t);
hipError_t launch_weight_zero_term(const uint32_t *, int, int, int, int, const float *, const float *, int, float *,
                                   hipStream_t);

// (x_bits, w_bits) pairs with specialised kernels: the twelve of the reference library
// (engine/mma_any/aq_bmma_impl/aq_bmma_w{2a2,...,8a8}.h).
#define ABQ_FOR_EACH_COMBO(F) \
    F(2, 2) F(4, 2) F(6, 2) F(8, 2) F(3, 3) F(8, 3) F(4, 4) F(8, 4) F(5, 5) F(6, 6) F(7, 7) F(8, 8)
#define ABQ_NUM_COMBOS 12

#define ABQ_DECL(Q, P)                                \
    void abq_mfma_register_##Q##_##P(KernelTable *);  \
    void abq_bcnt_register_##Q##_##P(KernelTable *);  \
    void abq_decode_register_##Q##_##P(KernelTable *); \
    void abq_decode_grouped_register_##Q##_##P(KernelTable *); \
    void abq_tiled_register_##Q##_##P(KernelTable *);  \
    void abq_tiled_grouped_register_##Q##_##P(KernelTable *);  \
    void abq_decode_tiled_register_##Q##_##P(KernelTable *); \
    void abq_decode_tiled_grouped_register_##Q##_##P(KernelTable *); \
    void abq_decode_tiled_f16_register_##Q##_##P(KernelTable *); \
    void abq_decode_tiled_grouped_dyn_register_##Q##_##P(KernelTable *);
ABQ_FOR_EACH_COMBO(ABQ_DECL)
#undef ABQ_DECL

struct Registry {
    KernelTable mfma[2 * ABQ_NUM_COMBOS];
    KernelTable bcnt[2 * ABQ_NUM_COMBOS];
    KernelTable decode[2 * ABQ_NUM_COMBOS];
    KernelTable decode_grouped[2 * ABQ_NUM_COMBOS];
    KernelTable tiled[2 * ABQ_NUM_COMBOS];
    KernelTable tiled_grouped[2 * ABQ_NUM_COMBOS];
    KernelTable decode_tiled[2 * ABQ_NUM_COMBOS];
    KernelTable decode_tiled_grouped[2 * ABQ_NUM_COMBOS];
    KernelTable decode_tiled_f16[2 * ABQ_NUM_COMBOS];
    KernelTable decode_tiled_grouped_dyn[2 * ABQ_NUM_COMBOS];
    Registry()
    {
        int i = 0;
#define ABQ_REG(Q, P)                                  \
    abq_mfma_register_##Q##_##P(&mfma[i]);             \
    abq_bcnt_register_##Q##_##P(&bcnt[i]);             \
    abq_decode_register_##Q##_##P(&decode[i]);         \
    abq_decode_grouped_register_##Q##_##P(&decode_grouped[i]); \
    abq_tiled_register_##Q##_##P(&tiled[i]);           \
    abq_tiled_grouped_register_##Q##_##P(&tiled_grouped[i]); \
    abq_decode_tiled_register_##Q##_##P(&decode_tiled[i]); \
    abq_decode_tiled_grouped_register_##Q##_##P(&decode_tiled_grouped[i]); \
    abq_decode_tiled_f16_register_##Q##_##P(&decode_tiled_f16[i]); \
    abq_decode_tiled_grouped_dyn_register_##Q##_##P(&decode_tiled_grouped_dyn[i]); \
    i += 2;
        ABQ_FOR_EACH_COMBO(ABQ_REG)
#undef ABQ_REG
    }
};

static const Registry &registry()
{
    static const Registry r;
    return r;
}

static const KernelTable *find_table(const KernelTable *tables, int x_bits, int w_bits, int is_signed)
{
    for (int i = 0; i < 2 * ABQ_NUM_COMBOS; ++i)
        if (tables[i].x_bits == x_bits && tables[i].w_bits == w_bits &&
            tables[i].is_signed == (is_signed ? 1 : 0))
            return &tables[i];
    return nullptr;
}

static thread_local int g_last_hip_error = 0;

static abq_status hip_status(hipError_t e)
{
    if (e == hipSuccess)
        return ABQ_OK;
    g_last_hip_error = (int)e;
    return e == hipErrorNoDevice || e == hipErrorInvalidDevice ? ABQ_ERR_NO_DEVICE : ABQ_ERR_LAUNCH;
}

// ---- tile tuple <-> kernel entry ---------------------------------------------------------

static void entry_to_config(const KernelEntry &e, int strategy, int x_bits, int w_bits,
                            int is_signed, int lpr_log2, abq_tile_config *c)
{
    c->x_bits = x_bits;
    c->w_bits = w_bits;
    c->is_signed = is_signed ? 1 : 0;
    if (strategy == ABQ_STRATEGY_BCNT) {
        const int lpr = 1 << lpr_log2;
        c->block_m = e.tm;
        c->block_n = e.wn * (64 / lpr);
        c->block_k = lpr * 128;
        c->warp_m = e.tm;
        c->warp_n = 64 / lpr;
        c->warp_k = lpr * 128;
        c->mma_m = 1;
        c->mma_n = 1;
        c->mma_k = 128;
        c->nstage = e.nstage; // passes whose loads a lane keeps in flight
    } else {
        // NSTAGE 4 (K-tiled layout, 128- or 64-element stages) and NSTAGE 3 (decode, 512- or 256-element steps)
        // carry their K step; the direct kernels step 4 plane words per lane group
        const int stepk = (e.nstage >= 3) ? e.kb : (64 / e.mi) * 4 * 32;
        c->block_m = e.mi * e.tm * e.wm;
        c->block_n = e.mi * e.tn * e.wn;
        c->block_k = stepk * e.wk;
        c->warp_m = e.mi * e.tm;
        c->warp_n = e.mi * e.tn;
        c->warp_k = stepk;
        c->mma_m = e.mi;
        c->mma_n = e.mi;
        c->mma_k = e.nstage == 5 ? 64 : 1024 / e.mi; // NSTAGE 5: the FP6 MFMA, 32x32x64
        c->nstage = e.nstage;
    }
}

static int strategy_of_mma(const abq_tile_config &c)
{
    if (c.mma_m == 1 && c.mma_n == 1 && c.mma_k == 128)
        return ABQ_STRATEGY_BCNT;
    if (c.mma_m == 16 && c.mma_n == 16 && c.mma_k == 64)
        return ABQ_STRATEGY_MFMA16;
    if (c.mma_m == 32 && c.mma_n == 32 && c.mma_k == 32)
        return ABQ_STRATEGY_MFMA32;
    if (c.mma_m == 32 && c.mma_n == 32 && c.mma_k == 64)
        return ABQ_STRATEGY_FP6;
    return ABQ_STRATEGY_AUTO;
}

// The FP6 route is exact when both operands are E2M3 numbers (magnitude <= 16 in units of 1/8:
// unsigned up to 4 bits, signed up to 5) and no partial sum can reach 2^24.
static bool fp6_eligible(int x_bits, int w_bits, int is_signed, int K)
{
    const int lim = is_signed ? 5 : 4;
    if (x_bits < 1 || w_bits < 1 || x_bits > lim || w_bits > lim)
        return false;
    const long mx = is_signed ? (1L << (x_bits - 1)) : (1L << x_bits) - 1;
    const long mw = is_signed ? (1L << (w_bits - 1)) : (1L << w_bits) - 1;
    return mx * mw * (long)K < (1L << 24);
}

static size_t fp6_bytes(int rows, int k) { return (size_t)rows * (k / 128) * 96; }

// Lanes per weight row for the popcount kernels: the power of two in [16, 64] that wastes
// the fewest lanes for this K (a row has K/128 sixteen-byte units).
static int best_lpr_log2(int K)
{
    const int units = K / 128;
    // A row of at most 64 units: the fewest lanes that cover it in one pass, every load of the row in flight at once
    // (K = 5120, 40 units: 64 lanes ahead of three passes of 16 by up to 20 % on the wide pairs, level on the narrow ones).
    if (units <= 64)
        return units <= 16 ? 4 : units <= 32 ? 5 : 6;
    int best = 6;
    double best_eff = 0;
    for (int l = 4; l <= 6; ++l) {
        const int lpr = 1 << l;
        const int iters = (units + lpr - 1) / lpr;
        const double eff = (double)units / (iters * lpr);
        if (eff > best_eff + 1e-9 || (eff > best_eff - 1e-9 && l > best)) {
            best_eff = eff;
            best = l;
        }
    }
    return best;
}

static int find_mfma_variant(const KernelTable &t, int mi, int tm, int tn, int wm, int wn, int wk)
{
    for (int i = 0; i < t.count; ++i) {
        const KernelEntry &e = t.entries[i];
        if (e.mi == mi && e.tm == tm && e.tn == tn && e.wm == wm && e.wn == wn && e.wk == wk)
            return i;
    }
    return -1;
}

// Default choice when the caller names no native tile (operands in the reference's plane layout).
//
// Decode-sized M (at most 16 rows): the VALU popcount kernel or the matrix-core decode kernel.  The popcount
// kernel works on the planes as they are and costs x_bits * w_bits * M AND + popcount pairs per 128 weights; the
// matrix-core kernel pays a bit-matrix transpose per 32 weights that grows with w_bits (steeply from 6 planes
// up) and nothing per row.  Measured on MI355X over the twelve bit pairs, M = 1, 2, 4, 8 and the LLaMA-7B
// shapes, the popcount kernel is the faster one while x_bits * w_bits * M stays at or below a bound that
// depends on w_bits: it wins every pair at M = 1 (by 2 to 52 %), the low products and the 6- to 8-bit weights at
// M = 2, and almost nothing from M = 4 up.  Above 16 rows: 32-row MFMA tiles.
// K elements per work item of the default decode kernel (512 or 256, see abq_gemm_decode.hip)
static const int kDefaultDecodeStep = 512;

static bool popcount_is_faster(int x_bits, int w_bits, int M)
{
    static const int bound[9] = { 0, 16, 16, 27, 32, 40, 100, 150, 200 }; // by w_bits
    return w_bits >= 1 && w_bits <= 8 && x_bits * w_bits * M <= bound[w_bits];
}

static void choose_default(int M, int N, int K, int x_bits, int w_bits, int *strategy, int *mi, int *tm, int *tn, int *wm,
                           int *wn, int *wk)
{
    if (M <= 16 && popcount_is_faster(x_bits, w_bits, M)) {
        *strategy = ABQ_STRATEGY_BCNT;
        *mi = 1; *tm = M <= 1 ? 1 : M <= 2 ? 2 : 4; *tn = 1; *wm = 1; *wn = 8; *wk = 1;
    } else if (M <= 16) {
        // sixteen waves split K, eight where both operands are at least 5 bits wide (the transposes of that many planes
        // in sixteen waves: W8A8 8 x 4096 x 4096 15.5 against 7.6 us, W6A6 9.9 against 6.7, W5A5 6.9 against 5.5) or K is
        // short (8192 x 1024: 10 - 15 % on every pair); measured over M = 3 ... 16 on five shapes
        *strategy = ABQ_STRATEGY_DECODE;
        *mi = 16; *tm = 1; *tn = 1; *wm = 1; *wn = 1; *wk = ((x_bits >= 5 && w_bits >= 5) || K <= 2048) ? 8 : 16;
    } else if (M <= 64 ? (N < 8192 || w_bits <= 4 || M <= 32)
                       : (w_bits < 8 && (M <= 128 || (M <= 256 && K >= 8192)) && N < 8192)) {
        // 17 to 128 rows: blocks of 16 rows whose waves split K (16-row MFMA tiles, two per wave), which fill the chip
        // where the 32-row tiles below leave most of it idle (W2A8 32 x 4096 x 4096: 8.7 against 22.4 us, W4A4
        // 64 x 4096 x 4096, the reference's own test shape: 12.9 against 32.7 us).  Up to 64 rows the workgroup is one
        // column of four waves (eight for long K) on 32 weight rows, above that two columns of two on 64 (up to 256
        // rows when K is long: 256 x 4096 x 11008 53.7 against 74.9 us).  Every block of rows transposes the weight
        // planes again, which costs by the plane: wide outputs of weights of five bits or more keep the 32-row tiles from
        // 33 rows on, 8-bit weights from 65 (W8A8 64 x 13824 x 5120: 55 against 101 us).
        *strategy = ABQ_STRATEGY_MFMA16;
        *mi = 16; *tm = 1; *tn = 2; *wm = 1;
        if (M <= 64) {
            *wn = 1; *wk = K >= 8192 ? 8 : 4;
        } else {
            *wn = 2; *wk = 2;
        }
    } else {
        *strategy = ABQ_STRATEGY_MFMA32;
        *mi = 32; *wm = 2; *wn = 2; *wk = 1;
        const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
        if (M > 64 && tiles128 >= 256) {
            *tm = 2; *tn = 2;
        } else if (M > 64 && w_bits < 8) {
            *tm = 1; *tn = 2;
        } else {
            *tm = 1; *tn = 1;
        }
    }
}

static abq_status resolve(const abq_tile_config *cfg, int x_bits, int w_bits, int is_signed, int M,
                          int N, int K, abq_gemm_state *st)
{
    const Registry &reg = registry();
    int strategy = cfg ? strategy_of_mma(*cfg) : ABQ_STRATEGY_AUTO;
    if (strategy == ABQ_STRATEGY_FP6) {
        if (cfg->nstage != 5 || cfg->warp_k != 128 || cfg->block_k != 128 || cfg->warp_m <= 0 || cfg->warp_n <= 0 ||
            cfg->warp_m % 32 || cfg->warp_n % 32 || cfg->block_m % cfg->warp_m || cfg->block_n % cfg->warp_n)
            return ABQ_ERR_UNSUPPORTED;
        if (!fp6_eligible(x_bits, w_bits, is_signed, K))
            return ABQ_ERR_UNSUPPORTED;
        int count = 0;
        const KernelEntry *es = fp6_entries(&count);
        int v = -1;
        for (int i = 0; i < count; ++i)
            if (es[i].tm == cfg->warp_m / 32 && es[i].tn == cfg->warp_n / 32 && es[i].wm == cfg->block_m / cfg->warp_m &&
                es[i].wn == cfg->block_n / cfg->warp_n)
                v = i;
        if (v < 0)
            return ABQ_ERR_UNSUPPORTED;
        const KernelEntry &e = es[v];
        const int bm = 32 * e.tm * e.wm, bn = 32 * e.tn * e.wn;
        const int mblocks = (M + bm - 1) / bm, npx = ((N + bn - 1) / bn + 7) / 8;
        st->strategy = strategy;
        st->variant = v;
        entry_to_config(e, strategy, x_bits, w_bits, is_signed, 0, &st->cfg);
        st->grid_dim = abq_dim3{ (unsigned)(8 * npx * mblocks), 1, 1 };
        st->block_dim = abq_dim3{ (unsigned)(64 * e.wm * e.wn * e.wk), 1, 1 };
        st->shared_mem_size = e.lds;
        return ABQ_OK;
    }
    const KernelTable *tm_ = find_table(reg.mfma, x_bits, w_bits, is_signed);
    const KernelTable *tb_ = find_table(reg.bcnt, x_bits, w_bits, is_signed);
    const KernelTable *td_ = find_table(reg.decode, x_bits, w_bits, is_signed);
    if (!tm_ || !tb_ || !td_) {
        // no specialised instantiation: run-time loop kernel, one activation row per grid row
        if (x_bits < 1 || x_bits > 16 || w_bits < 1 || w_bits > 16)
            return ABQ_ERR_UNSUPPORTED;
        if (M > 65535)
            return ABQ_ERR_TOO_LARGE;
        st->strategy = ABQ_STRATEGY_GENERIC;
        st->variant = 0;
        st->cfg = abq_tile_config{ x_bits, w_bits, is_signed ? 1 : 0, 1, 4, 2048, 1, 1, 2048, 1, 1, 32, 1 };
        st->grid_dim = abq_dim3{ (unsigned)((N + 3) / 4 > 65536 ? 65536 : (N + 3) / 4), (unsigned)M, 1 };
        st->block_dim = abq_dim3{ 256, 1, 1 };
        st->shared_mem_size = 0;
        return ABQ_OK;
    }

    int mi = 0, tm = 0, tn = 0, wm = 0, wn = 0, wk = 0;
    int lpr_log2 = best_lpr_log2(K);
    int decode_step = cfg ? cfg->warp_k : 0; // K elements per decode work item
    if (strategy == ABQ_STRATEGY_AUTO) {
        choose_default(M, N, K, x_bits, w_bits, &strategy, &mi, &tm, &tn, &wm, &wn, &wk);
        decode_step = kDefaultDecodeStep;
    } else if (strategy == ABQ_STRATEGY_BCNT) {
        mi = 1; tm = cfg->block_m; tn = 1; wm = 1; wn = 8; wk = 1;
        // block_k = lanes per row * 128; accept 16, 32 or 64 lanes, else keep the best fit
        const int lpr = cfg->block_k / 128;
        if (cfg->block_k % 128 == 0 && (lpr == 16 || lpr == 32 || lpr == 64))
            lpr_log2 = lpr == 16 ? 4 : lpr == 32 ? 5 : 6;
    } else {
        mi = cfg->mma_m;
        const int stepk = ((strategy == ABQ_STRATEGY_MFMA32 && cfg->nstage == 4) ||
                           (strategy == ABQ_STRATEGY_MFMA16 && (cfg->nstage == 3 || cfg->nstage == 6))) ? cfg->warp_k : (64 / mi) * 4 * 32;
        if (cfg->warp_m <= 0 || cfg->warp_n <= 0 || cfg->warp_m % mi || cfg->warp_n % mi ||
            cfg->block_m % cfg->warp_m || cfg->block_n % cfg->warp_n || cfg->warp_k != stepk ||
            cfg->block_k % stepk)
            return ABQ_ERR_UNSUPPORTED;
        tm = cfg->warp_m / mi; tn = cfg->warp_n / mi;
        wm = cfg->block_m / cfg->warp_m; wn = cfg->block_n / cfg->warp_n;
        wk = cfg->block_k / stepk;
        if (strategy == ABQ_STRATEGY_MFMA16 && cfg->nstage == 3)
            strategy = ABQ_STRATEGY_DECODE;
        if (strategy == ABQ_STRATEGY_MFMA16 && cfg->nstage == 6)
            strategy = ABQ_STRATEGY_DECODE_TILED;
        if (strategy == ABQ_STRATEGY_MFMA32 && cfg->nstage == 4)
            strategy = ABQ_STRATEGY_TILED;
    }

    if (strategy == ABQ_STRATEGY_TILED) {
        const KernelTable *tt_ = find_table(reg.tiled, x_bits, w_bits, is_signed);
        if (!tt_ || mi != 32)
            return ABQ_ERR_UNSUPPORTED;
        int v = -1;
        for (int i = 0; i < tt_->count; ++i) {
            const KernelEntry &t = tt_->entries[i];
            if (t.tm == tm && t.tn == tn && t.wm == wm && t.wn == wn && t.wk == wk && t.kb == cfg->warp_k)
                v = i;
        }
        if (v < 0)
            return ABQ_ERR_UNSUPPORTED;
        if (K >= (1 << 17))
            return ABQ_ERR_TOO_LARGE;
        const KernelEntry &e = tt_->entries[v];
        const int bm = 32 * e.tm * e.wm, bn = 32 * e.tn * e.wn;
        const int mblocks = (M + bm - 1) / bm, npx = ((N + bn - 1) / bn + 7) / 8;
        st->strategy = strategy;
        st->variant = v;
        entry_to_config(e, strategy, x_bits, w_bits, is_signed, 0, &st->cfg);
        st->grid_dim = abq_dim3{ (unsigned)(8 * npx * mblocks), 1, 1 };
        st->block_dim = abq_dim3{ (unsigned)(64 * e.wm * e.wn * e.wk), 1, 1 };
        st->shared_mem_size = e.lds ? e.lds : 2 * (size_t)(bm + bn) * (e.kb + 16) + (bm + bn) * 4;
        return ABQ_OK;
    }

    if (strategy == ABQ_STRATEGY_DECODE_TILED) {
        const KernelTable *tdt = find_table(reg.decode_tiled, x_bits, w_bits, is_signed);
        if (!tdt || mi != 16 || tm != 1 || wm != 1 || wn != 1)
            return ABQ_ERR_UNSUPPORTED;
        int v = -1;
        for (int i = 0; i < tdt->count; ++i)
            if (tdt->entries[i].tn == tn && tdt->entries[i].wk == wk && tdt->entries[i].kb == cfg->warp_k)
                v = i;
        if (v < 0)
            return ABQ_ERR_UNSUPPORTED;
        const KernelEntry &e = tdt->entries[v];
        const int xq = abq_padded_bits(x_bits); // width of the activation records the kernel reads
        const int mrows = decode_tiled_rows(e.wk, e.tn, M, K, xq);
        // byte offsets inside the kernel are 32 bits wide
        if (mrows == 0 || K >= (1 << 17) || (size_t)N * K * w_bits / 8 >= (1ull << 32) || (size_t)M * K * xq / 8 >= (1ull << 32) ||
            (M + mrows - 1) / mrows > 65535)
            return ABQ_ERR_TOO_LARGE;
        st->strategy = strategy;
        st->variant = v;
        entry_to_config(e, strategy, x_bits, w_bits, is_signed, 0, &st->cfg);
        st->grid_dim = abq_dim3{ (unsigned)(((N + 15) / 16 + e.tn - 1) / e.tn), (unsigned)((M + mrows - 1) / mrows), 1 };
        st->block_dim = abq_dim3{ (unsigned)(64 * e.wk), 1, 1 };
        st->shared_mem_size = decode_tiled_lds(e.wk, e.tn, mrows, K, xq);
        return ABQ_OK;
    }

    if (strategy == ABQ_STRATEGY_DECODE) {
        if (mi != 16 || tm != 1 || tn != 1 || wm != 1 || wn != 1)
            return ABQ_ERR_UNSUPPORTED;
        int v = -1;
        for (int i = 0; i < td_->count; ++i)
            if (td_->entries[i].wk == wk && td_->entries[i].kb == decode_step)
                v = i;
        if (v < 0)
            return ABQ_ERR_UNSUPPORTED;
        if (K >= (1 << 17) || (M + 15) / 16 > 65535)
            return ABQ_ERR_TOO_LARGE;
        const KernelEntry &e = td_->entries[v];
        const int tiles = (N + 15) / 16;
        int gx = tiles < 256 ? tiles : 256;
        if ((tiles + gx - 1) / gx > 8)
            gx = (tiles + 7) / 8;
        st->strategy = strategy;
        st->variant = v;
        entry_to_config(e, strategy, x_bits, w_bits, is_signed, 0, &st->cfg);
        st->grid_dim = abq_dim3{ (unsigned)gx, (unsigned)((M + 15) / 16), 1 };
        st->block_dim = abq_dim3{ (unsigned)(64 * e.wk), 1, 1 };
        st->shared_mem_size = 0; // sized at launch from M and K (dynamic LDS)
        return ABQ_OK;
    }

    if (strategy == ABQ_STRATEGY_BCNT) {
        int v = -1;
        // passes in flight: the tuple's NSTAGE; a library choice takes one pass per lane when that covers K, else three
        const int want_d = cfg && strategy_of_mma(*cfg) == ABQ_STRATEGY_BCNT ? cfg->nstage : (K / 128 <= (1 << lpr_log2) ? 1 : 3);
        for (int i = 0; i < tb_->count; ++i)
            if (tb_->entries[i].tm == tm && tb_->entries[i].nstage == want_d)
                v = i;
        if (v < 0)
            return ABQ_ERR_UNSUPPORTED;
        const KernelEntry &e = tb_->entries[v];
        const int rows_per_wg = e.wn * (64 >> lpr_log2);
        const int mb = M < e.tm ? M : e.tm;
        const size_t lds = (size_t)x_bits * mb * (K / 32) * 4 + 1024;
        if ((M + e.tm - 1) / e.tm > 65535 || lds > 160 * 1024 || (size_t)N * (K / 32) * 4 >= (1ull << 32))
            return ABQ_ERR_TOO_LARGE;
        st->strategy = strategy;
        st->variant = v;
        entry_to_config(e, strategy, x_bits, w_bits, is_signed, lpr_log2, &st->cfg);
        st->grid_dim = abq_dim3{ (unsigned)((N + rows_per_wg - 1) / rows_per_wg), (unsigned)((M + e.tm - 1) / e.tm), 1 };
        st->block_dim = abq_dim3{ (unsigned)(64 * e.wn), 1, 1 };
        st->shared_mem_size = lds;
        st->reserved[0] = lpr_log2;
        return ABQ_OK;
    }

    const int v = find_mfma_variant(*tm_, mi, tm, tn, wm, wn, wk);
    if (v < 0)
        return ABQ_ERR_UNSUPPORTED;
    const KernelEntry &e = tm_->entries[v];
    // The signed path scales both operands to the top of the byte: |acc| <= K * 2^14.
    if (K >= (1 << 17))
        return ABQ_ERR_TOO_LARGE;
    const int bm = e.mi * e.tm * e.wm, bn = e.mi * e.tn * e.wn;
    if ((M + bm - 1) / bm > 65535)
        return ABQ_ERR_TOO_LARGE;
    st->strategy = strategy;
    st->variant = v;
    entry_to_config(e, strategy, x_bits, w_bits, is_signed, 0, &st->cfg);
    st->grid_dim = abq_dim3{ (unsigned)((N + bn - 1) / bn), (unsigned)((M + bm - 1) / bm), 1 };
    st->block_dim = abq_dim3{ (unsigned)(64 * e.wm * e.wn * e.wk), 1, 1 };
    const int acc = e.mi == 16 ? 4 : 16;
    st->shared_mem_size = e.wk > 1 ? (size_t)e.wm * e.wn * (e.wk - 1) * (e.tm * e.tn * acc + e.tm + e.tn) * 64 * 4 : 0;
    return ABQ_OK;
}

} // namespace abq

using namespace abq;

extern "C" {

const char *abq_status_string(abq_status s)
{
    switch (s) {
    case ABQ_OK: return "ok";
    case ABQ_ERR_INVALID_ARG: return "invalid argument";
    case ABQ_ERR_BAD_K: return "K must be >= 128 and a multiple of 128";
    case ABQ_ERR_UNSUPPORTED: return "unsupported bit combination, tile tuple or option";
    case ABQ_ERR_NOT_INITIALIZED: return "state not initialised";
    case ABQ_ERR_LAUNCH: return "HIP launch failed";
    case ABQ_ERR_NO_DEVICE: return "no usable HIP device";
    case ABQ_ERR_TOO_LARGE: return "size exceeds a documented limit";
    }
    return "unknown status";
}

int abq_last_hip_error(void) { return g_last_hip_error; }
int abq_version(void) { return ABQ_VERSION; }

// ---- packing -----------------------------------------------------------------------------

static abq_status check_pack(const void *in, const void *out, int rows, int k, int bits)
{
    if (!in || !out || rows <= 0 || k <= 0 || bits < 1 || bits > 32)
        return ABQ_ERR_INVALID_ARG;
    if (k % 32 != 0)
        return ABQ_ERR_BAD_K;
    return ABQ_OK;
}

abq_status abq_pack_i32(const int32_t *in, uint32_t *planes, int rows, int k, int bits, void *stream)
{
    abq_status s = check_pack(in, planes, rows, k, bits);
    if (s != ABQ_OK)
        return s;
    return hip_status(launch_pack_i32(in, planes, rows, k, bits, (hipStream_t)stream));
}

abq_status abq_pack_u4(const uint32_t *in, uint32_t *planes, int rows, int k, int bits, void *stream)
{
    abq_status s = check_pack(in, planes, rows, k, bits);
    if (s != ABQ_OK)
        return s;
    return hip_status(launch_pack_u4(in, planes, rows, k, bits, (hipStream_t)stream));
}

abq_status abq_pack_f16(const void *in_f16, const float *scale_dev, uint32_t *planes, int rows,
                        int k, int bits, void *stream)
{
    abq_status s = check_pack(in_f16, planes, rows, k, bits);
    if (s != ABQ_OK)
        return s;
    if (!scale_dev)
        return ABQ_ERR_INVALID_ARG;
    return hip_status(launch_pack_f16(in_f16, scale_dev, planes, rows, k, bits, (hipStream_t)stream));
}

abq_status abq_pack_f16_tiled(const void *in_f16, const float *scale_dev, uint32_t *tiled, int rows, int k, int bits,
                              void *stream)
{
    abq_status s = check_pack(in_f16, tiled, rows, k, bits);
    if (s != ABQ_OK)
        return s;
    if (!scale_dev || bits > 8)
        return ABQ_ERR_INVALID_ARG;
    return hip_status(launch_pack_f16_tiled(in_f16, scale_dev, tiled, rows, k, bits, (hipStream_t)stream));
}

abq_status abq_pack_f16_fp6(const void *in_f16, const float *scale_dev, uint32_t *records, int rows, int k, int bits,
                            int is_signed, void *stream)
{
    abq_status s = check_pack(in_f16, records, rows, k, bits);
    if (s != ABQ_OK)
        return s;
    if (!scale_dev)
        return ABQ_ERR_INVALID_ARG;
    if (bits > (is_signed ? 5 : 4))
        return ABQ_ERR_UNSUPPORTED;
    if (k % 128 != 0)
        return ABQ_ERR_BAD_K;
    return hip_status(launch_pack_f16_fp6(in_f16, scale_dev, records, rows, k, bits, is_signed ? 1 : 0, (hipStream_t)stream));
}

// ---- names -------------------------------------------------------------------------------

abq_status abq_parse_kernel_name(const char *name, abq_tile_config *cfg, int *is_wmma)
{
    if (!name || !cfg)
        return ABQ_ERR_INVALID_ARG;
    const char *p = name;
    int wmma = 0;
    if (strncmp(p, "AqBWMMA_", 8) == 0) {
        wmma = 1;
        p += 8;
    } else if (strncmp(p, "AqBMMA_", 7) == 0) {
        p += 7;
    } else {
        return ABQ_ERR_INVALID_ARG;
    }
    abq_tile_config c;
    char sign[8] = { 0 };
    int consumed = 0;
    // 8x2xtrue_1x48x512_8x24x128_8x8x128_4
    if (sscanf(p, "%dx%dx%5[a-z]_%dx%dx%d_%dx%dx%d_%dx%dx%d_%d%n", &c.x_bits, &c.w_bits, sign,
               &c.block_m, &c.block_n, &c.block_k, &c.warp_m, &c.warp_n, &c.warp_k, &c.mma_m,
               &c.mma_n, &c.mma_k, &c.nstage, &consumed) != 13)
        return ABQ_ERR_INVALID_ARG;
    if (strcmp(sign, "true") == 0)
        c.is_signed = 1;
    else if (strcmp(sign, "false") == 0)
        c.is_signed = 0;
    else
        return ABQ_ERR_INVALID_ARG;
    const char *rest = p + consumed;
    if (*rest != '\0' && strcmp(rest, "_InitFn") != 0 && strcmp(rest, "_ExecFn") != 0)
        return ABQ_ERR_INVALID_ARG;
    *cfg = c;
    if (is_wmma)
        *is_wmma = wmma;
    return ABQ_OK;
}

abq_status abq_format_kernel_name(const abq_tile_config *c, int is_wmma, char *buf, size_t n)
{
    if (!c || !buf || n == 0)
        return ABQ_ERR_INVALID_ARG;
    int w = snprintf(buf, n, "%s_%dx%dx%s_%dx%dx%d_%dx%dx%d_%dx%dx%d_%d", is_wmma ? "AqBWMMA" : "AqBMMA",
                     c->x_bits, c->w_bits, c->is_signed ? "true" : "false", c->block_m, c->block_n,
                     c->block_k, c->warp_m, c->warp_n, c->warp_k, c->mma_m, c->mma_n, c->mma_k,
                     c->nstage);
    return (w < 0 || (size_t)w >= n) ? ABQ_ERR_TOO_LARGE : ABQ_OK;
}

// Native tile space: popcount entries for 16/32/64 lanes per row, the decode kernel, the direct MFMA kernels,
// the LDS-staged kernels, the FP6 kernel, the decode kernel on K-tiled operands.
static int native_config(int x_bits, int w_bits, int is_signed, int index, abq_tile_config *cfg)
{
    const Registry &reg = registry();
    const KernelTable *tb = find_table(reg.bcnt, x_bits, w_bits, is_signed);
    const KernelTable *tm = find_table(reg.mfma, x_bits, w_bits, is_signed);
    const KernelTable *td = find_table(reg.decode, x_bits, w_bits, is_signed);
    const KernelTable *tt = find_table(reg.tiled, x_bits, w_bits, is_signed);
    const KernelTable *tdt = find_table(reg.decode_tiled, x_bits, w_bits, is_signed);
    if (!tb || !tm || !td || !tt)
        return 0;
    int n = 0;
    // returns true when `index` falls into the next `count` entries
    auto in = [&](int count) {
        const bool hit = cfg && index >= n && index < n + count;
        n += count;
        return hit;
    };
    if (in(tb->count * 3))
        entry_to_config(tb->entries[(index - (n - tb->count * 3)) / 3], ABQ_STRATEGY_BCNT, x_bits, w_bits, is_signed,
                        4 + (index - (n - tb->count * 3)) % 3, cfg);
    if (in(td->count))
        entry_to_config(td->entries[index - (n - td->count)], ABQ_STRATEGY_DECODE, x_bits, w_bits, is_signed, 0, cfg);
    if (in(tm->count)) {
        const KernelEntry &e = tm->entries[index - (n - tm->count)];
        entry_to_config(e, e.mi == 16 ? ABQ_STRATEGY_MFMA16 : ABQ_STRATEGY_MFMA32, x_bits, w_bits, is_signed, 0, cfg);
    }
    // (entries that want row sums handed in stand behind the kernel of the same tuple, at the end: no tuples of their own)
    int tt_count = tt->count;
    while (tt_count > 0 && (tt->entries[tt_count - 1].flags & kNeedsRowSums))
        --tt_count;
    if (in(tt_count))
        entry_to_config(tt->entries[index - (n - tt_count)], ABQ_STRATEGY_TILED, x_bits, w_bits, is_signed, 0, cfg);
    if (fp6_eligible(x_bits, w_bits, is_signed, 128)) {
        int nfp6 = 0;
        const KernelEntry *es = fp6_entries(&nfp6);
        if (in(nfp6))
            entry_to_config(es[index - (n - nfp6)], ABQ_STRATEGY_FP6, x_bits, w_bits, is_signed, 0, cfg);
    }
    if (tdt && in(tdt->count))
        entry_to_config(tdt->entries[index - (n - tdt->count)], ABQ_STRATEGY_DECODE_TILED, x_bits, w_bits, is_signed, 0, cfg);
    return n;
}

int abq_native_config_count(int x_bits, int w_bits, int is_signed)
{
    return native_config(x_bits, w_bits, is_signed, -1, nullptr);
}

abq_status abq_native_config_get(int x_bits, int w_bits, int is_signed, int index, abq_tile_config *cfg)
{
    if (!cfg || index < 0)
        return ABQ_ERR_INVALID_ARG;
    const int n = native_config(x_bits, w_bits, is_signed, index, cfg);
    if (n == 0)
        return ABQ_ERR_UNSUPPORTED;
    return index < n ? ABQ_OK : ABQ_ERR_INVALID_ARG;
}

// ---- GEMM --------------------------------------------------------------------------------

static void apply_tuned(abq_gemm_state *st);

abq_status abq_gemm_init(const abq_tile_config *cfg, int x_bits, int w_bits, int is_signed,
                         const uint32_t *X, const uint32_t *W, int M, int N, int K, void *D,
                         const void *C, int bias, int out_kind, abq_gemm_state *state)
{
    if (!state)
        return ABQ_ERR_INVALID_ARG;
    memset(state, 0, sizeof(*state));
    if (cfg) {
        x_bits = cfg->x_bits;
        w_bits = cfg->w_bits;
        is_signed = cfg->is_signed;
    }
    if (!X || !W || !D || M <= 0 || N <= 0 || K <= 0)
        return ABQ_ERR_INVALID_ARG;
    if (x_bits < 1 || w_bits < 1)
        return ABQ_ERR_INVALID_ARG;
    if (bias) // the reference asserts !bias (engine/mma_any/aq_bmma_op.h:79)
        return ABQ_ERR_UNSUPPORTED;
    if (K < 128 || K % 128 != 0)
        return ABQ_ERR_BAD_K;
    if (out_kind < ABQ_OUT_I32 || out_kind > ABQ_OUT_F16_TENSOR_F32SCALE)
        return ABQ_ERR_INVALID_ARG;
    if ((out_kind == ABQ_OUT_F16_TENSOR || out_kind == ABQ_OUT_F16_TENSOR_F32SCALE) && !C)
        return ABQ_ERR_INVALID_ARG;
    if ((long)M * N >= (1L << 31) || (long)M * (K / 32) >= (1L << 31) || (long)N * (K / 32) >= (1L << 31))
        return ABQ_ERR_TOO_LARGE;

    abq_status s = resolve(cfg, x_bits, w_bits, is_signed, M, N, K, state);
    if (s != ABQ_OK)
        return s;
    state->M = M;
    state->N = N;
    state->K = K;
    state->X = X;
    state->W = W;
    state->C = C;
    state->D = D;
    state->bias = 0;
    state->out_kind = out_kind;
    state->auto_chosen = (!cfg || strategy_of_mma(*cfg) == ABQ_STRATEGY_AUTO) ? 1 : 0;
    state->init_success = 1;
    apply_tuned(state); // a measured best tile for this shape on plane operands, if the table holds one
    return ABQ_OK;
}

// ---- K-tiled layout, workspace -------------------------------------------------------------

static size_t planes_bytes(int rows, int k, int bits) { return (size_t)bits * rows * (k / 32) * 4; }

// Large tiles against the 128x128 tile, from sweeps over M = 256 .. 16384 and the LLaMA widths on MI355X.
// A large tile (one workgroup per compute unit) moves fewer bytes from L2 per MFMA and runs `gain` times
// faster per output element once the chip is kept full over several rounds of workgroups (`gain1` while
// the grid is a single round), but its grid is quantised: a last round that is partly empty costs up to
// a full one.  Two 128x128 workgroups share a compute unit and one of them alone runs nearly twice as
// fast, so that grid degrades smoothly with its tile count.
struct LargeTile {
    int tm, tn, wm, wn; // MFMA tiles per wave, waves along M and N
    double gain1, gain;
};

// Cost of the shape on the 128x128 tile, in units of the time two co-resident 128x128 workgroups take.
static double cost_128x128(int M, int N)
{
    const long t = (long)((M + 127) / 128) * ((N + 127) / 128);
    return t <= 256 ? 0.6 : t <= 512 ? 1.0 : (double)t / 512.0;
}

static double cost_large(const LargeTile &c, int M, int N)
{
    const int bm = 32 * c.tm * c.wm, bn = 32 * c.tn * c.wn;
    const long t = (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    const double area = (double)bm * bn / (2.0 * 128 * 128);
    if (t <= 256)
        return area / c.gain1;
    // workgroups do not run in lockstep, so a short last round partly hides behind the others; not so for the
    // 256x256 tiles, whose workgroups are few and long
    const double frac = (double)(t % 256) / 256.0;
    const double tail = area >= 2.0 ? (frac > 0 ? 1.0 : 0.0) : (1.5 * frac < 1.0 ? 1.5 * frac : 1.0);
    return ((double)(t / 256) + tail) * area / c.gain;
}

// Index in `entries` of the best large tile that beats the 128x128 tile by a margin, or -1.
static int pick_large_tile(const KernelEntry *entries, int count, const LargeTile *cands, int ncands, int M, int N)
{
    double best = 0.97 * cost_128x128(M, N);
    int pick = -1;
    for (int k = 0; k < ncands; ++k) {
        const double cost = cost_large(cands[k], M, N);
        if (cost >= best)
            continue;
        for (int i = 0; i < count; ++i)
            if (entries[i].tm == cands[k].tm && entries[i].tn == cands[k].tn && entries[i].wm == cands[k].wm &&
                entries[i].wn == cands[k].wn && entries[i].wk == 1 && entries[i].kb == 128) {
                best = cost;
                pick = i;
            }
    }
    return pick;
}

// Large tiles of the int8 kernels per operand pair (sweep with the grouped tile mapping): for the pairs
// below 16 bits together only 256x256 (eight waves of 64x128) beats 128x128, by 5-7 % once its grid
// is a whole number of rounds; signed W8A8 gains 20 % from 256x128 as soon as that fills the chip.
// Pairs of widths made of several fields keep the thresholds below.
static int large_tiles_int8(int x_bits, int w_bits, int is_signed, const LargeTile **out)
{
    static const LargeTile wide_n[] = { { 2, 4, 4, 2, 1.06, 1.06 } };
    static const LargeTile w8a8[] = { { 2, 2, 4, 2, 1.20, 1.20 } };
    const bool field = (x_bits == 2 || x_bits == 4 || x_bits == 8) && (w_bits == 2 || w_bits == 4 || w_bits == 8);
    (void)is_signed; // (the staged kernel serves unsigned 8-bit operands too, given their row sums)
    if (x_bits == 8 && w_bits == 8) {
        *out = w8a8;
        return 1;
    }
    if (field && x_bits >= w_bits) {
        *out = wide_n;
        return 1;
    }
    return 0;
}

// Picks the tiled-kernel tile for a shape.  Pairs with a cost model (large_tiles_int8) weigh their large
// tiles against 128x128 once the shape has 200 tiles of 128x128; everything else goes by the thresholds
// below (measured on MI355X, LLaMA shapes): smaller tiles win by filling the chip.
static abq_status switch_to_tiled(abq_gemm_state *st)
{
    const Registry &reg = registry();
    const abq_tile_config &c = st->cfg;
    const KernelTable *tt = find_table(reg.tiled, c.x_bits, c.w_bits, c.is_signed);
    if (!tt)
        return ABQ_ERR_UNSUPPORTED;
    // candidates in order of preference: { TM, TN, waves along M, waves along N, workgroups needed }
    // (pairs without a cost model: the 256x256 tile of eight 64x128 waves only for operands of 16 bits together,
    // on grids of several workgroups per compute unit)
    static const int order[][5] = { { 2, 4, 4, 2, 600 }, { 2, 2, 4, 2, 250 }, { 2, 2, 2, 2, 200 }, { 2, 1, 2, 2, 400 },
                                    { 1, 1, 2, 2, 0 } };
    // signed W8A8 below 200 tiles of 128x128: the staged kernel's 256x128 tile pays as soon as it covers about two
    // thirds of the compute units
    const bool staged = c.x_bits == 8 && c.w_bits == 8;
    int pick = -1;
    const LargeTile *cands = nullptr;
    const int ncands = large_tiles_int8(c.x_bits, c.w_bits, c.is_signed, &cands);
    const bool modelled = ncands > 0 && (long)((st->M + 127) / 128) * ((st->N + 127) / 128) >= 200;
    if (modelled)
        pick = pick_large_tile(tt->entries, tt->count, cands, ncands, st->M, st->N);
    for (const auto &o : order) {
        if (modelled && 32 * o[0] * o[2] * 32 * o[1] * o[3] > 128 * 128)
            continue; // the large tiles have been weighed against 128x128 above
        if (o[1] == 4 && c.x_bits + c.w_bits < 16)
            continue;
        const int bm = 32 * o[0] * o[2], bn = 32 * o[1] * o[3];
        const long tiles = (long)((st->M + bm - 1) / bm) * ((st->N + bn - 1) / bn);
        // (signed W8A8, which keeps its one-group tiles on small grids: 128x64 from one workgroup per compute unit,
        // 512 x 4096 x 4096 844 against 794 TOPS on 64x64)
        // (and both 128x128 and 128x64 from 160 workgroups: more than 256 of the smaller tile, whose stages fill a compute
        // unit's LDS, are a second round on part of the chip: 256 x 11008 x 4096 28.1 on 128x128 against 35.4 us on 128x64,
        // 768 x 4096 x 4096 29.2 against 32.1; 128 x 11008 x 4096 22.0 on 128x64 against 25.9 on 64x64, 384 x 4096 x 4096 21.2
        // against 21.9; 256 x 4096 x 4096, 128 workgroups of 128x64, stays on 64x64: 16.2)
        const long need = (staged && o[0] == 2 && o[1] == 2 && o[2] == 4) ? 160
                          : (staged && o[0] == 2 && o[1] == 2 && o[2] == 2) ? 160
                          : (staged && o[0] == 2 && o[1] == 1)              ? 160
                                                                            : o[4];
        for (int i = 0; i < tt->count; ++i)
            if (tt->entries[i].tm == o[0] && tt->entries[i].tn == o[1] && tt->entries[i].kb == 128 && tt->entries[i].wk == 1 &&
                tt->entries[i].wm == o[2] && tt->entries[i].wn == o[3] && tiles >= need && pick < 0)
                pick = i;
    }
    if (pick < 0)
        return ABQ_ERR_UNSUPPORTED;
    {
        // Small grids on the staged kernel.  What bounds them is the LDS traffic per MFMA (every byte of a tile is
        // written into LDS once and read by two waves) and the chain of latencies per K tile, not the matrix cores:
        // below 200 tiles of 128x128, two groups of waves per workgroup split K (half the K loop's trips for the same
        // tile), and where an activation row is the longer record the tile is laid along N (64x128: 12 instead of
        // 18 KB per K tile for W2A8), also up to 400 tiles, where 128x128 leaves part of the chip idle.  Sweep over
        // W2A8 and W4A4, M = 256 .. 2048 on the LLaMA-7B widths: 5-12 % below 200 tiles, 2-9 % on 64x128 up to 400
        // (W2A2 7-12 %, W4A8 1-5 %; W8A8, whose tiles are all LDS traffic, -5 .. +4 %: left as it was).
        const long t128 = (long)((st->M + 127) / 128) * ((st->N + 127) / 128);
        const long n64x64 = (long)((st->M + 63) / 64) * ((st->N + 63) / 64);
        const bool along_n = c.x_bits > c.w_bits;
        int want[5] = { 0, 0, 2, 2, 0 }; // TM, TN, waves along M and N, K groups
        if (tt->entries[pick].lds != 0 && t128 < 200 && c.x_bits + c.w_bits < 16) {
            want[4] = 2;
            want[0] = n64x64 <= 256 ? 1 : along_n ? 1 : 2; // 64x64 up to one workgroup per compute unit
            want[1] = n64x64 <= 256 ? 1 : along_n ? 2 : 1;
            // The stages of these tiles fill most of a compute unit's LDS: more than 256 workgroups of the 64x128 (128x64)
            // tile are a second round on part of the chip, and the 128x128 tile with the same split, one round below 200
            // tiles, is ahead (256 x 11008 x 4096: W4A8 23.2 against 30.2 us, W2A8 22.1 against 24.0, W4A4 22.3 against 24.3;
            // 768 x 4096 x 4096: W4A8 24.5 against 29.7).
            if ((long)((st->M + 32 * want[0] * 2 - 1) / (32 * want[0] * 2)) * ((st->N + 32 * want[1] * 2 - 1) / (32 * want[1] * 2)) > 256)
                want[0] = want[1] = 2;
        } else if (tt->entries[pick].lds != 0 && t128 <= 256 && c.x_bits + c.w_bits < 16) {
            // exactly one round of 128x128 tiles: that tile with the split (1024 x 4096 x 11008: W2A8 1725 against 1611
            // TOPS on 64x128, W4A4 1686 against 1530 on 128x128; on K = 4096 level with the best)
            want[4] = 2;
            want[0] = 2;
            want[1] = 2;
        } else if (tt->entries[pick].lds != 0 && along_n && t128 < 400 && tt->entries[pick].tm * tt->entries[pick].wm <= 4 &&
                   tt->entries[pick].tn * tt->entries[pick].wn <= 4) {
            want[4] = 1;
            want[0] = 1;
            want[1] = 2;
        }
        // W8A8 on long K, up to one round of its 128x64 tile: that tile with the split (512 x 4096 x 11008 41.0 against 43.9
        // us, 384 x 4096 x 11008 39.5 against 42.1; on K = 4096 within 3 %, in two rounds behind: left)
        if (!want[4] && staged && st->K >= 8192 && tt->entries[pick].lds != 0 && tt->entries[pick].tm == 2 && tt->entries[pick].tn == 1 &&
            tt->entries[pick].wm == 2 && tt->entries[pick].wn == 2 && (long)((st->M + 127) / 128) * ((st->N + 63) / 64) <= 256) {
            want[0] = 2;
            want[1] = 1;
            want[4] = 2;
        }
        for (int i = 0; want[4] && i < tt->count; ++i) {
            const KernelEntry &e = tt->entries[i];
            if (e.lds != 0 && e.tm == want[0] && e.tn == want[1] && e.wm == want[2] && e.wn == want[3] && e.wk == want[4] && e.kb == 128)
                pick = i;
        }
    }
    abq_tile_config cfg;
    entry_to_config(tt->entries[pick], ABQ_STRATEGY_TILED, c.x_bits, c.w_bits, c.is_signed, 0, &cfg);
    abq_gemm_state tmp = *st;
    const abq_status rc = resolve(&cfg, c.x_bits, c.w_bits, c.is_signed, st->M, st->N, st->K, &tmp);
    if (rc != ABQ_OK)
        return rc;
    *st = tmp;
    return ABQ_OK;
}

// Picks the FP6 kernel's tile for a shape: the largest tile that still yields enough workgroups.
static abq_status switch_to_fp6(abq_gemm_state *st)
{
    const abq_tile_config &c = st->cfg;
    if (!fp6_eligible(c.x_bits, c.w_bits, c.is_signed, st->K))
        return ABQ_ERR_UNSUPPORTED;
    if (st->group_size) {
        // group scales: one scale per K tile, i.e. groups of 128.  Below 256 tiles of 128x128 (one round): 128x64, the
        // smallest tile with two MFMA tiles per wave; above, 256x128 runs 6 % faster than 128x128 where its
        // rounds of workgroups come out even (sweep of the three tiles over M = 512 .. 16384 and the LLaMA
        // widths: the choice is within 0.1 % of the best tile on average, 4 % at worst)
        if (st->group_size != 128)
            return ABQ_ERR_UNSUPPORTED;
        int gcount = 0;
        const KernelEntry *ge = fp6_grouped_entries(&gcount);
        const long t128 = (long)((st->M + 127) / 128) * ((st->N + 127) / 128);
        static const LargeTile grouped_large[] = { { 2, 2, 4, 2, 1.06, 1.06 } };
        const int large = st->auto_chosen && t128 >= 300 ? pick_large_tile(ge, gcount, grouped_large, 1, st->M, st->N) : -1;
        int gpick = -1;
        for (int i = 0; i < gcount; ++i) {
            const int bm = 32 * ge[i].tm * ge[i].wm, bn = 32 * ge[i].tn * ge[i].wn;
            if (!st->auto_chosen ? (bm == c.block_m && bn == c.block_n && 32 * ge[i].tm == c.warp_m)
                                 : large >= 0 ? i == large
                                              : ((t128 >= 256 && bm == 128 && bn == 128) || (t128 < 256 && bm == 128 && bn == 64)))
                gpick = i;
        }
        if (gpick < 0)
            return ABQ_ERR_UNSUPPORTED;
        const KernelEntry &e = ge[gpick];
        const int bm = 32 * e.tm * e.wm, bn = 32 * e.tn * e.wn;
        const int xb_ = c.x_bits, wb_ = c.w_bits, sg_ = c.is_signed;
        entry_to_config(e, ABQ_STRATEGY_FP6, xb_, wb_, sg_, 0, &st->cfg);
        st->strategy = ABQ_STRATEGY_FP6;
        st->variant = gpick;
        st->grid_dim = abq_dim3{ (unsigned)(8 * (((st->N + bn - 1) / bn + 7) / 8) * ((st->M + bm - 1) / bm)), 1, 1 };
        st->block_dim = abq_dim3{ (unsigned)(64 * e.wm * e.wn * e.wk), 1, 1 };
        st->shared_mem_size = e.lds;
        return ABQ_OK;
    }
    int count = 0;
    const KernelEntry *es = fp6_entries(&count);
    // 128x128 (two workgroups per compute unit) from 200 tiles up unless 256x128 is estimated ahead, below that the
    // smaller ones: { TM, TN, waves along M, waves along N, workgroups needed }
    static const int order[][5] = { { 2, 2, 2, 2, 200 }, { 2, 1, 2, 2, 256 }, { 1, 1, 2, 2, 0 } };
    // (at the clock the chip sustains the 256x128 tile runs 6-10 % ahead of 128x128 wherever its rounds of workgroups
    // come out even: weighed by the same model as on the int8 route)
    static const LargeTile fp6_large[] = { { 2, 2, 4, 2, 1.07, 1.07 } };
    int pick = (long)((st->M + 127) / 128) * ((st->N + 127) / 128) >= 200 ? pick_large_tile(es, count, fp6_large, 1, st->M, st->N) : -1;
    for (const auto &o : order) {
        if (pick >= 0)
            break;
        const int bm = 32 * o[0] * o[2], bn = 32 * o[1] * o[3];
        const long tiles = (long)((st->M + bm - 1) / bm) * ((st->N + bn - 1) / bn);
        for (int i = 0; i < count; ++i)
            if (es[i].tm == o[0] && es[i].tn == o[1] && es[i].wm == o[2] && es[i].wn == o[3] && tiles >= o[4] && pick < 0)
                pick = i;
    }
    if (pick < 0)
        return ABQ_ERR_UNSUPPORTED;
    abq_tile_config cfg;
    entry_to_config(es[pick], ABQ_STRATEGY_FP6, c.x_bits, c.w_bits, c.is_signed, 0, &cfg);
    abq_gemm_state tmp = *st;
    const abq_status rc = resolve(&cfg, c.x_bits, c.w_bits, c.is_signed, st->M, st->N, st->K, &tmp);
    if (rc != ABQ_OK)
        return rc;
    *st = tmp;
    return ABQ_OK;
}

// Moves a state whose tile was the library's choice onto the matrix-core decode kernel for plane operands.
static abq_status switch_to_decode(abq_gemm_state *st)
{
    const abq_tile_config &c = st->cfg;
    const KernelTable *td = find_table(registry().decode, c.x_bits, c.w_bits, c.is_signed);
    if (!td)
        return ABQ_ERR_UNSUPPORTED;
    for (int i = 0; i < td->count; ++i) {
        if (td->entries[i].wk != 16 || td->entries[i].kb != kDefaultDecodeStep)
            continue;
        abq_tile_config cfg;
        entry_to_config(td->entries[i], ABQ_STRATEGY_DECODE, c.x_bits, c.w_bits, c.is_signed, 0, &cfg);
        abq_gemm_state tmp = *st;
        const abq_status rc = resolve(&cfg, c.x_bits, c.w_bits, c.is_signed, st->M, st->N, st->K, &tmp);
        if (rc == ABQ_OK)
            *st = tmp;
        return rc;
    }
    return ABQ_ERR_UNSUPPORTED;
}

// Between 17 and 128 rows on prepared operands the decode kernel, run over blocks of 16 rows that each stream the
// weights again (from L2 after the first), is weighed against the 64 x 64 tile of the prefill kernel, whose time
// does not depend on M there but is a whole K loop of 0.23 us per K tile on a quarter of the compute units.  Both
// estimates are fits to a sweep of W2A8, W4A8, W8A8, W4A4 and W2A2 over M = 24 ... 128 and the LLaMA-7B widths on
// MI355X (microseconds; MB = 10^6 bytes of weights plus of the activations all workgroups of a block stage); the
// decode kernel is taken when it is estimated at least 10 % ahead, which on the sweep never picks the slower kernel
// by more than 5 % and gains up to 2.7 x (W4A4 64 x 4096 x 4096: 5.7 against 9.5 us).
constexpr int kDecodeTiledBlocksWaves = 8, kDecodeTiledBlocksTiles = 2;
static bool decode_tiled_pays(int x_bits, int w_bits, int M, int N, int K)
{
    if (M <= 16)
        return true;
    if (M > 128 || !(x_bits == 2 || x_bits == 4 || x_bits == 8) || !(w_bits == 2 || w_bits == 4 || w_bits == 8))
        return false; // (the instances that walk several blocks of rows exist for operands of one field)
    const int mrows = decode_tiled_rows(kDecodeTiledBlocksWaves, kDecodeTiledBlocksTiles, M, K, x_bits);
    if (mrows == 0)
        return false;
    const double blocks = (M + mrows - 1) / mrows;
    const double w_mb = (double)N * K * w_bits / 8e6;
    const double x_mb = (double)((N + 16 * kDecodeTiledBlocksTiles - 1) / (16 * kDecodeTiledBlocksTiles)) * mrows * K * x_bits / 8e6;
    // 8-bit activations: a block costs by the bytes it moves; narrower ones by the elements it multiplies (0.037 us per
    // 10^6 for 16 rows: W4A4 64 x 4096 x 4096 5.7, 128 x 11008 x 4096 18.0; W2A2 128 x 4096 x 4096 7.5), half as much
    // again for weights of 4 bits on long K
    const double melems = (double)N * K / 1e6 * mrows / 16.0;
    const double per_block = x_bits == 8 ? 0.11 * (w_mb + x_mb) + 0.5 : 0.037 * melems * (w_bits >= 4 && K > 8192 ? 1.5 : 1.0);
    const double decode_us = (x_bits == 8 ? 0.8 : 2.7) + blocks * per_block;
    // (all pairs but W8A8 run that tile with two groups of waves that split K: 5.0 + 0.145 us per K tile on weights
    // that come from HBM, e.g. W2A8 64 x 4096 x 4096 9.7, 64 x 4096 x 11008 17.5 us)
    const long tiles64 = (long)((M + 63) / 64) * ((N + 63) / 64);
    const int kt = K / 128;
    const double tiled_us = (x_bits + w_bits < 16 ? 5.0 + 0.145 * kt : 2.3 + 0.23 * kt) * (tiles64 > 256 ? 1.35 : 1.0);
    return decode_us < 0.9 * tiled_us;
}

// Decode-sized GEMM with both operands K-tiled: the decode kernel built for that layout, if it exists for the
// pair.  Variant by shape (measured on MI355X, W2A8, LLaMA-7B widths): sixteen waves with one weight load each
// in flight while a compute unit holds at most two workgroups; with more tiles than that, eight waves with two
// loads each (twice the workgroups fit a compute unit).
// reserved[4]: bit 0 / bit 1: the K-tiled 8-bit records of X / W hold code - 128 (abq_gemm_set_biased_records)
static bool biased_x(const abq_gemm_state *st) { return (st->reserved[4] & 1) != 0; }
static bool biased_w(const abq_gemm_state *st) { return (st->reserved[4] & 2) != 0; }
// reserved[4] bit 2: the K-tiled activation records are those of the next single-field width
// (abq_relayout_planes_padded), which is how the decode kernel on prepared operands reads activations of 3, 5, 6 or
// 7 bits (abq_gemm_set_padded_activations)
static bool padded_x(const abq_gemm_state *st) { return (st->reserved[4] & 4) != 0; }
static bool one_field(int bits) { return bits == 2 || bits == 4 || bits == 8; }
// Width of the activation records the decode kernel on prepared operands reads for a pair.
static int decode_tiled_x_bits(int x_bits) { return abq_padded_bits(x_bits); }
// Whether that kernel can read the state's activations as they are declared: planes (converted by exec), records of
// one field, or padded records for the widths of several fields.
static bool decode_tiled_x_ok(const abq_gemm_state *st, int x_layout)
{
    if (x_layout != ABQ_LAYOUT_TILED)
        return true; // (a declaration of padded records says nothing about planes or fp16)
    return one_field(st->cfg.x_bits) ? true : padded_x(st);
}
static bool decode_tiled_x_ok(const abq_gemm_state *st) { return decode_tiled_x_ok(st, st->x_layout); }

// Planes an operand arrives in: as many as its codes have bits, which abq_gemm_set_value_bits may have declared fewer
// than the state's (record) width.
static int x_plane_bits(const abq_gemm_state *st) {
    return st->reserved[2] > 0 && st->reserved[2] < st->cfg.x_bits ? st->reserved[2] : st->cfg.x_bits;
}
static int w_plane_bits(const abq_gemm_state *st) {
    return st->reserved[3] > 0 && st->reserved[3] < st->cfg.w_bits ? st->reserved[3] : st->cfg.w_bits;
}

// Unsigned 8-bit records on the decode kernel of prepared operands: codes up to 255 are fed as value - 128 and need
// the other operand's row sums (abq_gemm_set_row_sums); records declared to hold narrower codes
// (abq_gemm_set_value_bits: padded records) are fed as they are.  flip_x / flip_w: which operands are flipped.
static void decode_tiled_flips(const abq_gemm_state *st, int *flip_x, int *flip_w)
{
    const abq_tile_config &c = st->cfg;
    *flip_x = !c.is_signed && c.x_bits == 8 && (st->reserved[2] == 0 || st->reserved[2] == 8);
    *flip_w = !c.is_signed && c.w_bits == 8 && (st->reserved[3] == 0 || st->reserved[3] == 8);
}

// Whether that kernel can run the state as it stands: the sums are there, and two 8-bit operands are either both
// flipped or both not (there is no instance for a mix).
static bool decode_tiled_flips_ok(const abq_gemm_state *st)
{
    int fx, fw;
    decode_tiled_flips(st, &fx, &fw);
    if (biased_x(st) || biased_w(st))
        return false; // biased records are read by the prefill kernel only
    if (!decode_tiled_x_ok(st))
        return false; // activation records of several fields: the prefill kernel reads those
    if (fx && !st->w_row_sums)
        return false;
    if (fw && !st->x_row_sums)
        return false;
    if (!st->cfg.is_signed && st->cfg.x_bits == 8 && st->cfg.w_bits == 8 && fx != fw)
        return false;
    return true;
}

static abq_status switch_to_decode_tiled(abq_gemm_state *st, bool one_tile = false)
{
    const abq_tile_config &c = st->cfg;
    const KernelTable *tdt = find_table(registry().decode_tiled, c.x_bits, c.w_bits, c.is_signed);
    if (!tdt || tdt->count == 0 || !decode_tiled_flips_ok(st))
        return ABQ_ERR_UNSUPPORTED;
    const int tiles = (st->N + 15) / 16;
    const int steps = (st->K / 128 * c.w_bits + 3) / 4;
    // long K with one or two rows: three loads per wave in flight instead of three rounds of one (4.4 against 4.8 us
    // at K = 11008); with more rows the activation traffic comes first and one load at a time is as fast.  Several
    // blocks of 16 rows (M > 16): eight waves on two tiles, so that a workgroup's activations serve twice the weights.
    const bool row_blocks = st->M > 16;
    // Nine to sixteen rows: the activations a workgroup stages (every workgroup all of them) outweigh the weights of
    // one tile, so a workgroup takes several tiles: three on wide outputs, two on long K (W2A8 at 16 rows, 11008 x 4096:
    // 5.4 against 6.2 us; 4096 x 11008: 6.5 against 9.1).
    // (one_tile: the caller needs an instance of one tile per workgroup, the ones that quantise fp16 activations)
    const bool many_rows = !one_tile && !row_blocks && st->M > 8 && (tiles > 512 || steps > 32);
    const int want_t = row_blocks ? kDecodeTiledBlocksTiles : many_rows ? (tiles > 512 ? 3 : 2) : 1;
    const int want_wk = row_blocks ? kDecodeTiledBlocksWaves : many_rows ? 16 : tiles > 512 ? 8 : 16;
    // (8-bit weights keep one load in flight: W8A8 4096 x 4096 at one row 5.3 against 6.5 us, 4096 x 11008 10.2 against 11.7)
    const int want_d = row_blocks || many_rows ? 1 : tiles > 512 ? 2 : (steps > 32 && st->M <= 2 && c.w_bits < 8) ? 3 : 1;
    int pick = -1;
    if (one_field(c.w_bits)) {
        for (int i = 0; i < tdt->count; ++i) {
            const KernelEntry &e = tdt->entries[i];
            if (e.tn == want_t && e.wk == want_wk && e.kb == (512 / c.w_bits) * want_d)
                pick = i;
        }
    } else {
        // weights of several fields (gemm_decode_fields; warp K of the entry = 128 x loads in flight per wave), up to 16
        // rows.  Sixteen waves with two loads each, except 3-bit weights on outputs that give a compute unit more than
        // two workgroups: eight waves with four (W3A3 11008 x 4096 at one row 7.9 against 8.6 us; from 5 bits up the
        // kernel is bound by the work per field and sixteen waves stay ahead: W5A5 12.0 against 15.5, W7A7 17.7
        // against 20.6).
        if (row_blocks)
            return ABQ_ERR_UNSUPPORTED;
        const int wk = (tiles > 512 && c.w_bits == 3) ? 8 : 16, d = wk == 8 ? 4 : 2;
        for (int i = 0; i < tdt->count; ++i)
            if (tdt->entries[i].wk == wk && tdt->entries[i].kb == 128 * d)
                pick = i;
    }
    if (pick < 0)
        return ABQ_ERR_UNSUPPORTED;
    abq_tile_config cfg;
    entry_to_config(tdt->entries[pick], ABQ_STRATEGY_DECODE_TILED, c.x_bits, c.w_bits, c.is_signed, 0, &cfg);
    abq_gemm_state tmp = *st;
    const abq_status rc = resolve(&cfg, c.x_bits, c.w_bits, c.is_signed, st->M, st->N, st->K, &tmp);
    if (rc != ABQ_OK)
        return rc;
    *st = tmp;
    return ABQ_OK;
}

// Group scales on a decode-sized GEMM whose operands are (or are about to be declared) both prepared: whether the
// decode kernel of that layout has a group-scale variant for the pair that fits this shape.
// The same weighing for the group-scale variant (one tile per workgroup, two with the SiLU gate), against the
// group-scale prefill kernel, whose smallest grids (128 x 64 tiles) take 4 + 0.42 us per K tile whatever M is and
// 1 + 0.6 x 1.45 per K tile once they exceed one workgroup per compute unit.  Fits to a sweep of W2A8, W4A8 and W4A4
// with zero points over M = 24 ... 128 on the LLaMA-7B linears (4096 x 4096, QKV, gate + up with the gate fused,
// down); taken when estimated 10 % ahead: W2A8 32 x 4096 x 4096 8.3 against 17 us, 32 x 4096 x 11008 24 against 38;
// the wide outputs of the 8-bit activations stay on the prefill kernel.
static bool decode_tiled_grouped_pays(int x_bits, int w_bits, int M, int N, int K, int act, int group_size)
{
    if (M <= 16)
        return true;
    if (M > 128)
        return false;
    const int t = act ? 2 : 1;
    const int mrows = decode_tiled_grouped_rows(16, t, M, K, x_bits);
    if (mrows == 0)
        return false;
    const double blocks = (M + mrows - 1) / mrows;
    const double w_mb = (double)N * K * w_bits / 8e6;
    const double x_mb = (double)((N + 16 * t - 1) / (16 * t)) * mrows * K * x_bits / 8e6;
    const double per_block = x_bits == 8 ? 0.165 * (w_mb + x_mb) : 0.11 * (w_mb + x_mb) + 0.7;
    const double decode_us = 1.0 + blocks * per_block;
    // (up to one workgroup per compute unit the prefill kernel's waves split K: 4 + 0.42 us per K tile on weights that
    // come from HBM, W2A8 64 x 4096 x 4096 17.4, 64 x 4096 x 11008 38.2 us)
    // (groups of 128, up to one 64x64 workgroup per compute unit: that tile with the split, 5 + 0.26 us per K tile:
    // 64 x 4096 x 4096 12.9, 64 x 4096 x 11008 26.8 us)
    const long wgs = (long)((N + 63) / 64) * ((M + 127) / 128), wgs64 = (long)((N + 63) / 64) * ((M + 63) / 64);
    const double tiled_us = group_size == 128 && wgs64 <= 256 ? 5.0 + 0.26 * (K / 128)
                            : wgs > 256                        ? 1.0 + 0.6 * 1.45 * (K / 128)
                                                               : 4.0 + 0.42 * (K / 128);
    return decode_us < 0.9 * tiled_us;
}

static bool decode_tiled_grouped_fits(const abq_gemm_state *st, int group_size, int act)
{
    const abq_tile_config &c = st->cfg;
    const KernelTable *t = find_table(registry().decode_tiled_grouped, c.x_bits, c.w_bits, c.is_signed);
    return t && t->count > 0 && st->auto_chosen && (group_size == 128 || group_size == 64) && (!act || st->N % 32 == 0) &&
           decode_tiled_grouped_rows(16, act ? 2 : 1, st->M, st->K, c.x_bits, group_size) != 0 &&
           decode_tiled_grouped_pays(c.x_bits, c.w_bits, st->M, st->N, st->K, act, group_size);
}

// Moves a state with group scales onto the tiled kernel's group-scale variants.
static abq_status pick_grouped_tiled(abq_gemm_state *state)
{
    if (state->x_layout == ABQ_LAYOUT_FP6 || state->w_layout == ABQ_LAYOUT_FP6 || state->strategy == ABQ_STRATEGY_FP6)
        return switch_to_fp6(state); // the FP6 kernel's group-scale variants
    if (state->strategy != ABQ_STRATEGY_TILED) {
        if (!state->auto_chosen)
            return ABQ_ERR_UNSUPPORTED;
        const abq_status rc = switch_to_tiled(state);
        if (rc != ABQ_OK)
            return rc;
    }
    const abq_tile_config &c = state->cfg;
    const KernelTable *tg = find_table(registry().tiled_grouped, c.x_bits, c.w_bits, c.is_signed);
    if (!tg)
        return ABQ_ERR_UNSUPPORTED;
    // entries with a fixed LDS size are the staged kernel's: one scale per K tile, i.e. groups of 128 only;
    // it is preferred where both kernels have the tile (they come later in the table)
    auto usable = [&](const KernelEntry &e) { return e.lds == 0 || state->group_size == 128; };
    auto block_m = [](const KernelEntry &e) { return e.mi * e.tm * e.wm; };
    auto block_n = [](const KernelEntry &e) { return e.mi * e.tn * e.wn; };
    int pick = -1;
    if (state->auto_chosen) {
        // The fold of the int32 tiles into fp32 bounds these kernels more than the tile traffic does, so tile
        // sizes from 128x128 up run within a few percent of each other (sweep over M = 256 .. 16384 and the
        // LLaMA widths): 128x128 once it fills the chip, below that 128x64, then 64x64.  With activations of
        // at most 4 bits three workgroups of 128x64 fit a compute unit and stay ahead up to 400 tiles.  (8-bit activations:
        // from the first tile past one round, 384 x 11008 x 4096 = 258 tiles: W2A8 40.3 against 46.9 us on 128x64.)
        const long t128 = (long)((state->M + 127) / 128) * ((state->N + 127) / 128);
        // W8A8 has the staged kernel at 128x64 only, and that runs 7-9 % ahead of the register-staged 128x128
        // (16384 x 4096 x 4096 / x 11008, 2048 x 12288 x 4096: 1098 / 1146 / 1038 against 1027 / 1038 / 1004 TOPS).
        const bool both8 = c.x_bits == 8 && c.w_bits == 8;
        const int order[][3] = { { 128, 128, both8 ? 1 << 30 : c.x_bits <= 4 ? 400 : 257 }, { 128, 64, 64 }, { 64, 64, 0 } };
        for (const auto &o : order) {
            if (pick >= 0 || t128 < o[2])
                continue;
            for (int i = 0; i < tg->count; ++i) // the last match: the staged kernel's entry where there is one
                if (usable(tg->entries[i]) && block_m(tg->entries[i]) == o[0] && block_n(tg->entries[i]) == o[1] &&
                    tg->entries[i].wk == 1)
                    pick = i;
        }
        // Grids of at most one 128x64 workgroup per compute unit: the tile whose two groups of waves split K (its
        // stages fill a compute unit's LDS, so beyond 256 workgroups it would run in two rounds).  W2A8 with zero
        // points: 4096 x 4096 64-512 rows 16-19 us against 19-21, 4096 x 11008 37-45 against 47-53, QKV up to 128
        // rows 17.5 against 20.3; QKV at 192 rows (384 workgroups) 33 against 29: not taken there.
        // Wider outputs of at most 64 rows, activations wider than the weights: the same along N (64x128: gate + up of
        // LLaMA-7B, 22016 wide, at 32-64 rows 19.4 against 28.7 us).
        const bool one_round = (long)((state->M + 127) / 128) * ((state->N + 63) / 64) <= 256;
        const bool along_n = !one_round && c.x_bits > c.w_bits && state->M <= 64 && (state->N + 127) / 128 <= 256;
        // Otherwise, up to one round of 128x128 tiles, that tile with the split (1024 x 4096 x 11008: 73 against 85 us,
        // 768 x 4096 x 4096 27.3 against 29.3; 320 workgroups, 1024 x 5120 x 5120: 68 against 57, not taken).
        const bool one_round_128 = !one_round && !along_n && (long)((state->M + 127) / 128) * ((state->N + 127) / 128) <= 256;
        if (one_round || along_n || one_round_128)
            for (int i = 0; i < tg->count; ++i)
                if (usable(tg->entries[i]) && tg->entries[i].lds != 0 && block_m(tg->entries[i]) == (along_n ? 64 : 128) &&
                    block_n(tg->entries[i]) == (one_round ? 64 : 128) && tg->entries[i].wk == 2 &&
                    tg->entries[i].wm * tg->entries[i].wn == 4)
                    pick = i;
        // Grids of at most one 64x64 workgroup per compute unit (batches of 17 to 64 rows up to QKV's width, 256 rows on
        // 4096 columns): that tile with the split, one MFMA tile per wave.  W2A8 with zero points, K = 4096: 12.6-13.5 us
        // against 15.5-17.1 on 128x64 with the split; K = 11008 at 64-256 rows 26.8-28.8 against 33.4-34.7.
        if ((long)((state->M + 63) / 64) * ((state->N + 63) / 64) <= 256)
            for (int i = 0; i < tg->count; ++i)
                if (usable(tg->entries[i]) && tg->entries[i].lds != 0 && block_m(tg->entries[i]) == 64 && block_n(tg->entries[i]) == 64 &&
                    tg->entries[i].wk == 2)
                    pick = i;
        // a measured best tile for this shape and group size comes before the rules above
        TunedTile t;
        if (tuning_find(c.x_bits, c.w_bits, c.is_signed, state->M, state->N, state->K, state->group_size, 1 << ABQ_LAYOUT_TILED, &t) &&
            t.cfg.nstage == 4 && t.cfg.warp_k > 0)
            for (int i = 0; i < tg->count; ++i)
                if (usable(tg->entries[i]) && block_m(tg->entries[i]) == t.cfg.block_m && block_n(tg->entries[i]) == t.cfg.block_n &&
                    tg->entries[i].mi * tg->entries[i].tm == t.cfg.warp_m && tg->entries[i].wk == t.cfg.block_k / t.cfg.warp_k)
                    pick = i;
    } else {
        const int wk = c.warp_k > 0 ? c.block_k / c.warp_k : 1;
        for (int i = 0; i < tg->count; ++i)
            if (usable(tg->entries[i]) && block_m(tg->entries[i]) == c.block_m && block_n(tg->entries[i]) == c.block_n &&
                tg->entries[i].wk == wk)
                pick = i;
    }
    if (pick < 0)
        return ABQ_ERR_UNSUPPORTED;
    const int xb_ = c.x_bits, wb_ = c.w_bits, sg_ = c.is_signed;
    entry_to_config(tg->entries[pick], ABQ_STRATEGY_TILED, xb_, wb_, sg_, 0, &state->cfg);
    state->variant = pick;
    {
        const KernelEntry &e = tg->entries[pick];
        const int bm = block_m(e), bn = block_n(e);
        state->grid_dim = abq_dim3{ (unsigned)(8 * (((state->N + bn - 1) / bn + 7) / 8) * ((state->M + bm - 1) / bm)), 1, 1 };
        state->block_dim = abq_dim3{ (unsigned)(64 * e.wm * e.wn * e.wk), 1, 1 };
        state->shared_mem_size = e.lds ? e.lds : 2 * (size_t)(bm + bn) * (e.kb + 16) + (bm + bn) * 4;
    }
    return ABQ_OK;
}

// Looks the state's GEMM up in the table of measured best tiles (abq_tuning.hip) and, if it holds a tile that runs
// on the operand layouts the state has now, moves the state to that tile.  Only states whose tile is the library's
// choice; group-scale states are looked up where their tile is picked (pick_grouped_tiled).
static void apply_tuned(abq_gemm_state *st)
{
    if (!st->auto_chosen || st->act || st->group_size || st->x_layout == ABQ_LAYOUT_F16)
        return;
    const abq_tile_config &c = st->cfg;
    const bool any_fp6 = st->x_layout == ABQ_LAYOUT_FP6 || st->w_layout == ABQ_LAYOUT_FP6;
    const bool any_tiled = st->x_layout == ABQ_LAYOUT_TILED || st->w_layout == ABQ_LAYOUT_TILED;
    const int mask = 1 << (any_fp6 ? ABQ_LAYOUT_FP6 : any_tiled ? ABQ_LAYOUT_TILED : ABQ_LAYOUT_PLANES);
    TunedTile t;
    if (!tuning_find(c.x_bits, c.w_bits, c.is_signed, st->M, st->N, st->K, 0, mask, &t))
        return;
    // the decode kernel on prepared operands converts activations that arrive as planes into the workspace, like the
    // prefill kernels; it cannot be chosen before there is one
    if (t.cfg.nstage == 6 && st->x_layout != ABQ_LAYOUT_TILED &&
        (!st->workspace || st->workspace_bytes < planes_bytes(st->M, st->K, c.x_bits)))
        return;
    if (t.cfg.nstage == 6 && !decode_tiled_flips_ok(st))
        return;
    if (memcmp(&t.cfg, &st->cfg, sizeof(abq_tile_config)) == 0)
        return;
    abq_gemm_state tmp = *st;
    if (resolve(&t.cfg, c.x_bits, c.w_bits, c.is_signed, st->M, st->N, st->K, &tmp) == ABQ_OK)
        *st = tmp;
}

abq_status abq_gemm_set_scales(abq_gemm_state *state, const float *x_scale, const float *w_scale,
                               int group_size)
{
    if (!state || !state->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (!x_scale || !w_scale)
        return ABQ_ERR_INVALID_ARG;
    if (group_size != 0) {
        // w_scale is [N][K / group_size]: the decode kernel with group scales for M <= 16 on plane
        // operands, the tiled kernel otherwise; both fold the scales inside the K loop
        const abq_tile_config &c = state->cfg;
        if (group_size != 64 && group_size != 128)
            return ABQ_ERR_UNSUPPORTED;
        if (state->out_kind != ABQ_OUT_F16_SCALED)
            return ABQ_ERR_INVALID_ARG;
        if (!c.is_signed && (c.x_bits == 8 || c.w_bits == 8))
            return ABQ_ERR_UNSUPPORTED;
        const abq_gemm_state before = *state; // a failed call leaves the state as it was
        state->group_size = group_size;
        if (state->strategy == ABQ_STRATEGY_BCNT && state->auto_chosen && state->M <= 16)
            switch_to_decode(state); // the popcount kernel has no group-scale epilogue
        // both operands prepared: the decode kernel of that layout has its own group-scale variant
        // (a state of 17 to 128 rows may sit on the prefill kernel because the plain decode kernel did not pay there)
        const bool both_tiled = state->x_layout == ABQ_LAYOUT_TILED && state->w_layout == ABQ_LAYOUT_TILED;
        bool decode_tiled_ok = (state->strategy == ABQ_STRATEGY_DECODE_TILED ||
                                (state->strategy == ABQ_STRATEGY_TILED && both_tiled && state->auto_chosen)) &&
                               decode_tiled_grouped_fits(state, group_size, state->act);
        if (decode_tiled_ok && state->strategy != ABQ_STRATEGY_DECODE_TILED)
            decode_tiled_ok = switch_to_decode_tiled(state) == ABQ_OK;
        const bool decode_ok = state->strategy == ABQ_STRATEGY_DECODE && state->auto_chosen && state->M <= 16 &&
                               state->x_layout == ABQ_LAYOUT_PLANES && state->w_layout == ABQ_LAYOUT_PLANES &&
                               decode_grouped_lds(state->M, state->K, group_size) != 0 &&
                               find_table(registry().decode_grouped, c.x_bits, c.w_bits, c.is_signed);
        if (decode_ok || decode_tiled_ok) {
            state->variant = 0;
        } else {
            const abq_status rc = pick_grouped_tiled(state);
            if (rc != ABQ_OK) {
                *state = before;
                return rc;
            }
        }
    } else if (state->group_size != 0) {
        return ABQ_ERR_INVALID_ARG; // a state switched to group scales stays there
    }
    state->x_scale = x_scale;
    state->w_scale = w_scale;
    state->group_size = group_size;
    return ABQ_OK;
}

abq_status abq_gemm_set_zero_points(abq_gemm_state *state, const float *x_zero, const float *w_zero,
                                    const int32_t *x_group_sums, const float *w_zero_term)
{
    if (!state || !state->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (state->group_size == 0) // only the group-scale kernel carries the correction terms
        return ABQ_ERR_UNSUPPORTED;
    const bool x_dynamic = state->x_layout == ABQ_LAYOUT_F16 && state->reserved[1] != 0; // sums and zero points made in the kernel
    if ((w_zero && !x_group_sums && !x_dynamic) || (x_zero && !w_zero_term) || (x_dynamic && state->reserved[1] == 2 && !w_zero_term))
        return ABQ_ERR_INVALID_ARG;
    state->x_zero = x_zero;
    state->w_zero = w_zero;
    state->x_group_sums = x_group_sums;
    state->w_zero_term = w_zero_term;
    return ABQ_OK;
}

abq_status abq_gemm_set_activation(abq_gemm_state *state, int act)
{
    if (!state || !state->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (act != ABQ_ACT_NONE && act != ABQ_ACT_SILU_GATE)
        return ABQ_ERR_INVALID_ARG;
    if (act == ABQ_ACT_SILU_GATE) {
        if (state->group_size == 0) // fused into the group-scale epilogues only
            return ABQ_ERR_UNSUPPORTED;
        if (state->N % 32 != 0)
            return ABQ_ERR_INVALID_ARG;
        // the decode kernel needs a gate tile and its up tile in one LDS pass
        if ((state->strategy == ABQ_STRATEGY_DECODE &&
             decode_grouped_lds(state->M, state->K, state->group_size) + (size_t)kDecodeGroupedWaves * 1024 > 160 * 1024) ||
            (state->strategy == ABQ_STRATEGY_DECODE_TILED && !decode_tiled_grouped_fits(state, state->group_size, act))) {
            const abq_status rc = pick_grouped_tiled(state);
            if (rc != ABQ_OK)
                return rc;
        }
    }
    state->act = act;
    return ABQ_OK;
}

abq_status abq_weight_zero_term(const uint32_t *w_planes, int n, int k, int bits, int is_signed,
                                const float *w_scale, const float *w_zero, int group_size,
                                float *w_zero_term, void *stream)
{
    if (!w_planes || !w_scale || !w_zero_term || n <= 0 || bits < 1 || bits > 8)
        return ABQ_ERR_INVALID_ARG;
    if (k < 128 || k % 128 != 0)
        return ABQ_ERR_BAD_K;
    if (group_size != 64 && group_size != 128)
        return ABQ_ERR_UNSUPPORTED;
    return hip_status(launch_weight_zero_term(w_planes, n, k, bits, is_signed, w_scale, w_zero, group_size,
                                              w_zero_term, (hipStream_t)stream));
}

abq_status abq_quant_pack_f16(const void *x_f16, int rows, int k, int bits, int symmetric, int layout,
                              uint32_t *planes, float *scale, float *zero, int32_t *group_sums,
                              int group_size, void *stream)
{
    if (!x_f16 || !planes || !scale || rows <= 0 || bits < 2 || bits > 8)
        return ABQ_ERR_INVALID_ARG;
    if (!symmetric && !zero)
        return ABQ_ERR_INVALID_ARG;
    if (layout < ABQ_LAYOUT_PLANES || layout > ABQ_LAYOUT_FP6)
        return ABQ_ERR_INVALID_ARG;
    if (layout == ABQ_LAYOUT_FP6 && bits > 5) // the codes are signed: magnitude at most 16
        return ABQ_ERR_UNSUPPORTED;
    if (k < 128 || k % 128 != 0)
        return ABQ_ERR_BAD_K;
    if (group_sums && group_size != 64 && group_size != 128)
        return ABQ_ERR_UNSUPPORTED;
    return hip_status(launch_quant_pack_rows(x_f16, planes, scale, zero, group_sums, rows, k, bits, symmetric ? 1 : 0,
                                             group_sums ? group_size : 128, layout, (hipStream_t)stream));
}

// ---- entry point that allocates nothing ----------------------------------------------------
//
// The layout conversions of abq_gemm_exec write into a workspace the caller brings.  Callers that cannot
// allocate one (code under HIP graph capture, serving loops, harnesses that forbid it) use
// abq_gemm_exec_static instead: the same launches with the workspace in a file-scope device array.  Every
// device the library runs on holds its own copy of the array, at its own address, until the process ends.
static __device__ __align__(256) unsigned char g_static_scratch[ABQ_STATIC_WORKSPACE_BYTES];

static const int kMaxDevices = 64;
static void *g_static_scratch_ptr[kMaxDevices]; // device address of the array, per device; null until asked for
static std::mutex g_static_scratch_mutex;

// Device address of the current device's copy of the array (the array's name is only a host-side handle).
static abq_status static_scratch_address(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return hip_status(e);
    if (dev < 0 || dev >= kMaxDevices)
        return ABQ_ERR_TOO_LARGE;
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (!g_static_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch));
        if (e != hipSuccess)
            return hip_status(e);
        if (!ptr)
            return ABQ_ERR_LAUNCH;
        g_static_scratch_ptr[dev] = ptr;
    }
    *out = g_static_scratch_ptr[dev];
    return ABQ_OK;
}

abq_status abq_gemm_exec_static(const abq_gemm_state *st, void *stream)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    // only the strategies on prepared layouts convert anything
    const bool converts = st->strategy == ABQ_STRATEGY_TILED || st->strategy == ABQ_STRATEGY_FP6 || st->strategy == ABQ_STRATEGY_DECODE_TILED;
    const size_t need = converts ? abq_gemm_workspace_bytes(st) : 0;
    if (need > (size_t)ABQ_STATIC_WORKSPACE_BYTES) {
        fprintf(stderr, "[ABQ][Error] abq_gemm_exec_static: this GEMM converts %zu bytes of operands, the static workspace holds %zu\n",
                need, (size_t)ABQ_STATIC_WORKSPACE_BYTES);
        return ABQ_ERR_TOO_LARGE;
    }
    abq_gemm_state local = *st;
    if (need) {
        void *ptr = nullptr;
        const abq_status rc = static_scratch_address(&ptr);
        if (rc != ABQ_OK)
            return rc;
        local.workspace = ptr;
        local.workspace_bytes = ABQ_STATIC_WORKSPACE_BYTES;
    }
    return abq_gemm_exec(&local, stream);
}

// Row sums of the operands of a state whose kernel wants them handed in (kNeedsRowSums): which are needed, which
// the caller has set, and where in the workspace (behind `converted` bytes of converted operands) those are put that
// the library can take itself, which it can only from an operand still in the reference's plane layout.
struct RowSumPlan {
    bool ok;             // every needed sum is set or can be taken into the workspace the state holds
    size_t x_off, w_off; // byte offsets into the workspace
    size_t bytes;        // workspace the sums need on top of the converted operands
};

static RowSumPlan row_sum_plan(const abq_gemm_state *st, size_t converted)
{
    const abq_tile_config &c = st->cfg;
    RowSumPlan p{ true, 0, 0, 0 };
    // which operands are fed as value - 128: every unsigned 8-bit one on the prefill kernel; on the decode kernel of
    // prepared operands those whose codes are not declared narrower
    int flip_x = c.x_bits == 8, flip_w = c.w_bits == 8;
    if (st->strategy == ABQ_STRATEGY_DECODE_TILED)
        decode_tiled_flips(st, &flip_x, &flip_w);
    const bool take_x = flip_w && !st->x_row_sums, take_w = flip_x && !st->w_row_sums;
    if ((take_x && st->x_layout != ABQ_LAYOUT_PLANES) || (take_w && st->w_layout != ABQ_LAYOUT_PLANES)) {
        p.ok = false; // a sum that is neither set nor to be had: the other kernel runs, and asks for nothing
        return p;
    }
    p.x_off = (converted + 255) / 256 * 256;
    p.w_off = p.x_off + (take_x ? ((size_t)st->M * 4 + 255) / 256 * 256 : 0);
    const size_t end = p.w_off + (take_w ? (size_t)st->N * 4 : 0);
    p.bytes = (take_x || take_w) ? end - converted : 0;
    if (p.bytes && (!st->workspace || converted + p.bytes > st->workspace_bytes))
        p.ok = false;
    return p;
}

// Whether the state's kernel is one that wants row sums handed in.
static bool wants_row_sums(const abq_gemm_state *st)
{
    if (st->group_size || st->cfg.is_signed || (st->cfg.x_bits != 8 && st->cfg.w_bits != 8))
        return false;
    if (st->strategy == ABQ_STRATEGY_DECODE_TILED) {
        int fx, fw;
        decode_tiled_flips(st, &fx, &fw);
        return fx || fw;
    }
    if (st->strategy != ABQ_STRATEGY_TILED)
        return false;
    const KernelTable *t = find_table(registry().tiled, st->cfg.x_bits, st->cfg.w_bits, 0);
    return t && st->variant >= 0 && st->variant < t->count && (t->entries[st->variant].flags & kNeedsRowSums);
}

abq_status abq_row_sums(const uint32_t *planes, int rows, int k, int bits, int32_t *sums, void *stream)
{
    if (!planes || !sums || rows <= 0 || bits < 1 || bits > 8)
        return ABQ_ERR_INVALID_ARG;
    if (k < 128 || k % 128 != 0)
        return ABQ_ERR_BAD_K;
    return hip_status(launch_row_sums(planes, sums, rows, k, bits, (hipStream_t)stream));
}

int abq_gemm_row_sums_ready(const abq_gemm_state *st)
{
    if (!st || !st->init_success || !wants_row_sums(st))
        return 0;
    const int xrec = st->strategy == ABQ_STRATEGY_DECODE_TILED ? decode_tiled_x_bits(st->cfg.x_bits) : st->cfg.x_bits;
    const size_t xb = st->x_layout == ABQ_LAYOUT_TILED ? 0 : planes_bytes(st->M, st->K, xrec);
    const size_t wb = st->w_layout == ABQ_LAYOUT_TILED ? 0 : planes_bytes(st->N, st->K, st->cfg.w_bits);
    return row_sum_plan(st, xb + wb).ok ? 1 : 0;
}

static abq_status switch_to_decode_tiled(abq_gemm_state *st, bool one_tile);
static bool decode_tiled_pays(int x_bits, int w_bits, int M, int N, int K);
static void apply_tuned(abq_gemm_state *st);

// A state on the prefill kernel whose operands are both prepared, once the decode kernel of that layout has become
// possible for it (row sums or value bits declared after the layouts): the move abq_gemm_set_operand_layout would
// have made.
static void reconsider_decode_tiled(abq_gemm_state *st)
{
    if (st->strategy == ABQ_STRATEGY_TILED && st->auto_chosen && !st->group_size && !st->act && st->x_layout == ABQ_LAYOUT_TILED &&
        st->w_layout == ABQ_LAYOUT_TILED && decode_tiled_pays(st->cfg.x_bits, st->cfg.w_bits, st->M, st->N, st->K))
        (void)switch_to_decode_tiled(st);
    apply_tuned(st);
}

abq_status abq_gemm_set_row_sums(abq_gemm_state *st, const int32_t *x_row_sums, const int32_t *w_row_sums)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    st->x_row_sums = x_row_sums;
    st->w_row_sums = w_row_sums;
    reconsider_decode_tiled(st);
    return ABQ_OK;
}

abq_status abq_gemm_set_value_bits(abq_gemm_state *st, int x_value_bits, int w_value_bits)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (x_value_bits < 1 || x_value_bits > st->cfg.x_bits || w_value_bits < 1 || w_value_bits > st->cfg.w_bits)
        return ABQ_ERR_INVALID_ARG;
    st->reserved[2] = x_value_bits;
    st->reserved[3] = w_value_bits;
    reconsider_decode_tiled(st);
    return ABQ_OK;
}

abq_status abq_gemm_set_padded_activations(abq_gemm_state *st, int padded)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (padded && one_field(st->cfg.x_bits))
        padded = 0; // records of one field are their own padding
    st->reserved[4] = (st->reserved[4] & ~4) | (padded ? 4 : 0);
    if (st->x_layout == ABQ_LAYOUT_TILED) {
        if (padded && st->strategy != ABQ_STRATEGY_DECODE_TILED) {
            reconsider_decode_tiled(st);
            if (st->strategy != ABQ_STRATEGY_DECODE_TILED) {
                st->reserved[4] &= ~4;
                return ABQ_ERR_UNSUPPORTED; // only the decode kernel on prepared operands reads such records
            }
        } else if (!padded && st->strategy == ABQ_STRATEGY_DECODE_TILED && !decode_tiled_x_ok(st)) {
            if (!st->auto_chosen)
                return ABQ_ERR_UNSUPPORTED;
            return st->group_size ? pick_grouped_tiled(st) : switch_to_tiled(st);
        }
    }
    return ABQ_OK;
}

abq_status abq_gemm_set_biased_records(abq_gemm_state *st, int x_biased, int w_biased)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if ((x_biased || w_biased) && (st->cfg.is_signed || st->cfg.x_bits != 8 || st->cfg.w_bits != 8 || st->group_size))
        return ABQ_ERR_UNSUPPORTED;
    if (x_biased && !w_biased)
        return ABQ_ERR_INVALID_ARG;
    st->reserved[4] = (x_biased ? 1 : 0) | (w_biased ? 2 : 0);
    if (w_biased && st->strategy == ABQ_STRATEGY_DECODE_TILED && st->auto_chosen)
        return switch_to_tiled(st); // biased records are read by the prefill kernel only
    return ABQ_OK;
}

abq_status abq_relayout_planes_biased(const uint32_t *planes, uint32_t *tiled, int rows, int k, void *stream)
{
    if (!planes || !tiled || rows <= 0)
        return ABQ_ERR_INVALID_ARG;
    if (k < 128 || k % 128 != 0)
        return ABQ_ERR_BAD_K;
    return hip_status(launch_relayout_planes_padded(planes, tiled, rows, k, 8, 8, 2, (hipStream_t)stream));
}

int abq_padded_bits(int bits) { return bits < 1 || bits > 8 ? 0 : bits <= 2 ? 2 : bits <= 4 ? 4 : 8; }

abq_status abq_relayout_planes_padded(const uint32_t *planes, uint32_t *tiled, int rows, int k, int bits, int is_signed,
                                      void *stream)
{
    if (!planes || !tiled || rows <= 0 || bits < 1 || bits > 8)
        return ABQ_ERR_INVALID_ARG;
    if (k < 128 || k % 128 != 0)
        return ABQ_ERR_BAD_K;
    return hip_status(launch_relayout_planes_padded(planes, tiled, rows, k, abq_padded_bits(bits), bits, is_signed ? 1 : 0,
                                                    (hipStream_t)stream));
}

int abq_folded_bits(int bits) { return bits < 1 || bits > 7 ? 0 : abq_padded_bits(bits + 1); }

abq_status abq_relayout_planes_folded(const uint32_t *planes, const float *w_zero, int group_size, uint32_t *tiled, int rows, int k,
                                      int bits, int is_signed, int *misfit_dev, void *stream)
{
    if (!planes || !w_zero || !tiled || rows <= 0 || bits < 1 || bits > 8 || group_size < 32 || group_size % 32 != 0)
        return ABQ_ERR_INVALID_ARG;
    if (k < 128 || k % 128 != 0 || k % group_size != 0 || (group_size > 128 && group_size % 128 != 0))
        return ABQ_ERR_BAD_K;
    if (!abq_folded_bits(bits))
        return ABQ_ERR_UNSUPPORTED; // 8-bit codes less their zero points need nine bits
    return hip_status(launch_relayout_planes_folded(planes, w_zero, group_size, tiled, rows, k, abq_folded_bits(bits), bits,
                                                    is_signed ? 1 : 0, misfit_dev, (hipStream_t)stream));
}

abq_status abq_gemm_exec(const abq_gemm_state *st, void *stream)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    const bool x_dynamic = st->x_layout == ABQ_LAYOUT_F16 && st->reserved[1] != 0; // the kernel takes the token scales itself
    if (st->out_kind == ABQ_OUT_F16_SCALED && ((!st->x_scale && !x_dynamic) || !st->w_scale))
        return ABQ_ERR_INVALID_ARG;
    GemmArgs a;
    a.X = st->X;
    a.W = st->W;
    a.D = st->D;
    a.C = st->C;
    a.x_scale = st->x_scale;
    a.w_scale = st->w_scale;
    a.M = st->M;
    a.N = st->N;
    a.K = st->K;
    a.KW = st->K / 32;
    a.out_kind = st->out_kind;
    a.group_size = st->group_size;
    a.lpr_log2 = st->reserved[0];
    a.act = st->act;
    a.w_zero = st->w_zero;
    a.x_zero = st->x_zero;
    a.x_group_sums = st->x_group_sums;
    a.w_zero_term = st->w_zero_term;
    a.x_pack_scale = st->x_pack_scale;
    a.x_dynamic = st->x_layout == ABQ_LAYOUT_F16 ? st->reserved[1] : 0;
    a.x_row_sums = nullptr; // (handed to a kernel only by the branches below that need them)
    a.w_row_sums = nullptr;
    decode_tiled_flips(st, &a.flip_x, &a.flip_w);
    const Registry &reg = registry();
    const abq_tile_config &c = st->cfg;
    hipError_t e;
    if (st->strategy == ABQ_STRATEGY_GENERIC) {
        e = launch_bcnt_generic(a, c.x_bits, c.w_bits, c.is_signed, (hipStream_t)stream);
    } else if (st->strategy == ABQ_STRATEGY_FP6) {
        // operands still in the reference layout are converted into the caller's workspace
        const size_t xb = st->x_layout == ABQ_LAYOUT_FP6 ? 0 : fp6_bytes(st->M, st->K);
        const size_t wb = st->w_layout == ABQ_LAYOUT_FP6 ? 0 : fp6_bytes(st->N, st->K);
        if (st->x_layout == ABQ_LAYOUT_TILED || st->w_layout == ABQ_LAYOUT_TILED)
            return ABQ_ERR_NOT_INITIALIZED;
        if (xb + wb > st->workspace_bytes || ((xb + wb) && !st->workspace))
            return ABQ_ERR_INVALID_ARG;
        char *ws = static_cast<char *>(st->workspace);
        if (xb) {
            e = launch_relayout_planes_fp6(st->X, reinterpret_cast<uint32_t *>(ws), st->M, st->K, x_plane_bits(st), c.is_signed,
                                           (hipStream_t)stream);
            if (e != hipSuccess)
                return hip_status(e);
            a.X = reinterpret_cast<const uint32_t *>(ws);
        }
        if (wb) {
            e = launch_relayout_planes_fp6(st->W, reinterpret_cast<uint32_t *>(ws + xb), st->N, st->K, w_plane_bits(st),
                                           c.is_signed, (hipStream_t)stream);
            if (e != hipSuccess)
                return hip_status(e);
            a.W = reinterpret_cast<const uint32_t *>(ws + xb);
        }
        int count = 0;
        const KernelEntry *es = st->group_size ? fp6_grouped_entries(&count) : fp6_entries(&count);
        if (st->variant < 0 || st->variant >= count)
            return ABQ_ERR_NOT_INITIALIZED;
        e = es[st->variant].launch(a, (hipStream_t)stream);
    } else if (st->strategy == ABQ_STRATEGY_TILED || st->strategy == ABQ_STRATEGY_DECODE_TILED) {
        // operands still in the reference layout are converted into the caller's workspace
        const bool x_f16 = st->x_layout == ABQ_LAYOUT_F16; // quantised inside the decode kernel
        // (the decode kernel reads activations of 3, 5, 6 or 7 bits as records of the next single-field width)
        const int xrec = st->strategy == ABQ_STRATEGY_DECODE_TILED ? decode_tiled_x_bits(c.x_bits) : c.x_bits;
        const size_t xb = (st->x_layout == ABQ_LAYOUT_TILED || x_f16) ? 0 : planes_bytes(st->M, st->K, xrec);
        const size_t wb = st->w_layout == ABQ_LAYOUT_TILED ? 0 : planes_bytes(st->N, st->K, c.w_bits);
        if (st->x_layout == ABQ_LAYOUT_FP6 || st->w_layout == ABQ_LAYOUT_FP6)
            return ABQ_ERR_NOT_INITIALIZED;
        if (st->strategy == ABQ_STRATEGY_DECODE_TILED ? !decode_tiled_x_ok(st) : (st->x_layout == ABQ_LAYOUT_TILED && padded_x(st)))
            return ABQ_ERR_INVALID_ARG; // records of the width this kernel does not read
        if (x_f16 && (st->strategy != ABQ_STRATEGY_DECODE_TILED ||
                      (x_dynamic ? st->group_size != 128 || (st->reserved[1] == 2 && !st->w_zero_term)
                                 : st->group_size != 0 || !st->x_pack_scale)))
            return ABQ_ERR_NOT_INITIALIZED;
        if (xb + wb > st->workspace_bytes || ((xb + wb) && !st->workspace))
            return ABQ_ERR_INVALID_ARG;
        char *ws = static_cast<char *>(st->workspace);
        // Unsigned W8A8 whose weights were prepared with the 128 already taken off (abq_relayout_planes_biased): the
        // activations are brought to the same form (converted that way here when they arrive as planes), and the
        // signed kernel of the same tile runs on them, handed both operands' row sums for the correction.
        const bool biased = st->strategy == ABQ_STRATEGY_TILED && biased_w(st);
        if (biased && (c.is_signed || c.x_bits != 8 || c.w_bits != 8 || st->group_size || wb || (!xb && !biased_x(st)) || (xb && biased_x(st))))
            return ABQ_ERR_INVALID_ARG;
        if (!biased && biased_x(st))
            return ABQ_ERR_INVALID_ARG; // biased activations only make sense against biased weights
        const KernelTable *t = find_table(st->strategy == ABQ_STRATEGY_DECODE_TILED
                                              ? (x_dynamic         ? reg.decode_tiled_grouped_dyn
                                                 : st->group_size ? reg.decode_tiled_grouped
                                                 : x_f16          ? reg.decode_tiled_f16
                                                                  : reg.decode_tiled)
                                          : st->group_size ? reg.tiled_grouped
                                                           : reg.tiled,
                                          c.x_bits, c.w_bits, c.is_signed);
        if (!t || st->variant < 0 || st->variant >= t->count)
            return ABQ_ERR_NOT_INITIALIZED;
        // Activations that arrive as planes and whose row sums a branch below will take from those planes: the
        // conversion's launch takes the sums as well (further workgroups of the same grid), where that branch puts them.
        bool x_sums_taken = false;
        if (xb && !c.is_signed && !st->x_row_sums) {
            const bool narrow = st->strategy == ABQ_STRATEGY_TILED && !biased && x_plane_bits(st) < c.x_bits && w_plane_bits(st) < c.w_bits;
            const bool wanted = biased ? true
                                : st->strategy == ABQ_STRATEGY_DECODE_TILED ? a.flip_w != 0
                                : !narrow && (t->entries[st->variant].flags & kNeedsRowSums) && c.w_bits == 8;
            const RowSumPlan plan = row_sum_plan(st, xb + wb);
            if (wanted && plan.ok) {
                e = launch_relayout_planes_padded(st->X, reinterpret_cast<uint32_t *>(ws), st->M, st->K, xrec, x_plane_bits(st), biased ? 2 : 0,
                                                  (hipStream_t)stream, reinterpret_cast<int *>(ws + plan.x_off));
                if (e != hipSuccess)
                    return hip_status(e);
                a.X = reinterpret_cast<const uint32_t *>(ws);
                x_sums_taken = true;
            }
        }
        if (xb && !x_sums_taken) {
            // (planes of fewer bits than the records: the codes are extended to the record's width)
            e = launch_relayout_planes_padded(st->X, reinterpret_cast<uint32_t *>(ws), st->M, st->K, xrec, x_plane_bits(st),
                                              biased ? 2 : (xrec != x_plane_bits(st) && c.is_signed ? 1 : 0), (hipStream_t)stream);
            if (e != hipSuccess)
                return hip_status(e);
            a.X = reinterpret_cast<const uint32_t *>(ws);
        }
        if (wb) {
            e = launch_relayout_planes_padded(st->W, reinterpret_cast<uint32_t *>(ws + xb), st->N, st->K, c.w_bits, w_plane_bits(st),
                                              w_plane_bits(st) != c.w_bits && c.is_signed ? 1 : 0, (hipStream_t)stream);
            if (e != hipSuccess)
                return hip_status(e);
            a.W = reinterpret_cast<const uint32_t *>(ws + xb);
        }
        int variant = st->variant;
        if (st->strategy == ABQ_STRATEGY_TILED && !c.is_signed && !biased && x_plane_bits(st) < c.x_bits && w_plane_bits(st) < c.w_bits) {
            // Unsigned codes that leave the top bit of their records clear are signed codes of the records' width as
            // well: the signed pair's kernel of the same tile reads them as they are (no value - 128, no row sums).
            const KernelTable *ts = find_table(st->group_size ? reg.tiled_grouped : reg.tiled, c.x_bits, c.w_bits, 1);
            const KernelEntry &want = t->entries[st->variant];
            for (int i = 0; ts && i < ts->count; ++i) {
                const KernelEntry &o = ts->entries[i];
                if ((o.lds != 0) == (want.lds != 0) && !(o.flags & kNeedsRowSums) && o.mi == want.mi && o.tm == want.tm && o.tn == want.tn &&
                    o.wm == want.wm && o.wn == want.wn && o.wk == want.wk && o.kb == want.kb && o.nstage == want.nstage)
                    return hip_status(o.launch(a, (hipStream_t)stream));
            }
        }
        if (biased) {
            const RowSumPlan plan = row_sum_plan(st, xb + wb);
            if (!plan.ok)
                return ABQ_ERR_INVALID_ARG; // both operands' sums are needed; the weights' must be set
            if (!st->x_row_sums && !x_sums_taken) {
                e = launch_row_sums(st->X, reinterpret_cast<int *>(ws + plan.x_off), st->M, st->K, x_plane_bits(st), (hipStream_t)stream);
                if (e != hipSuccess)
                    return hip_status(e);
            }
            a.x_row_sums = st->x_row_sums ? st->x_row_sums : reinterpret_cast<const int *>(ws + plan.x_off);
            a.w_row_sums = st->w_row_sums;
            // the signed pair's staged entry of the same tile
            const KernelTable *ts = find_table(reg.tiled, 8, 8, 1);
            const KernelEntry &want = t->entries[st->variant];
            const KernelEntry *run = nullptr;
            for (int i = 0; ts && i < ts->count; ++i) {
                const KernelEntry &o = ts->entries[i];
                if (o.lds != 0 && o.tm == want.tm && o.tn == want.tn && o.wm == want.wm && o.wn == want.wn && o.wk == want.wk && o.kb == want.kb)
                    run = &o;
            }
            if (!run)
                return ABQ_ERR_UNSUPPORTED; // a tile the staged kernel is not built for
            return hip_status(run->launch(a, (hipStream_t)stream));
        }
        if (st->strategy == ABQ_STRATEGY_DECODE_TILED && (a.flip_x || a.flip_w) && !c.is_signed) {
            // unsigned 8-bit codes on the decode kernel: the sums the caller set, or those of an operand that arrived
            // as planes, taken into the workspace behind its converted copy; there is no kernel to fall back to
            const RowSumPlan plan = row_sum_plan(st, xb + wb);
            if (!plan.ok || (c.x_bits == 8 && c.w_bits == 8 && a.flip_x != a.flip_w) || biased_x(st) || biased_w(st))
                return ABQ_ERR_INVALID_ARG;
            a.x_row_sums = st->x_row_sums;
            a.w_row_sums = st->w_row_sums;
            if (a.flip_w && !st->x_row_sums) {
                e = x_sums_taken ? hipSuccess
                                 : launch_row_sums(st->X, reinterpret_cast<int *>(ws + plan.x_off), st->M, st->K, x_plane_bits(st), (hipStream_t)stream);
                if (e != hipSuccess)
                    return hip_status(e);
                a.x_row_sums = reinterpret_cast<const int *>(ws + plan.x_off);
            }
            if (a.flip_x && !st->w_row_sums) {
                e = launch_row_sums(st->W, reinterpret_cast<int *>(ws + plan.w_off), st->N, st->K, w_plane_bits(st), (hipStream_t)stream);
                if (e != hipSuccess)
                    return hip_status(e);
                a.w_row_sums = reinterpret_cast<const int *>(ws + plan.w_off);
            }
        } else if (t->entries[variant].flags & kNeedsRowSums) {
            // An unsigned 8-bit operand is fed as value - 128 and the other operand's row sums put the result right.
            // The sums the caller set are taken; those of an operand still in planes are taken here, into the
            // workspace behind the converted copies, if it has the room.  Otherwise the kernel of the same tile
            // that gathers the sums itself runs.
            const bool need_x = c.w_bits == 8, need_w = c.x_bits == 8;
            const RowSumPlan plan = row_sum_plan(st, xb + wb);
            if (plan.ok) {
                if (need_x && !st->x_row_sums && !x_sums_taken) {
                    e = launch_row_sums(st->X, reinterpret_cast<int *>(ws + plan.x_off), st->M, st->K, x_plane_bits(st), (hipStream_t)stream);
                    if (e != hipSuccess)
                        return hip_status(e);
                }
                if (need_w && !st->w_row_sums) {
                    e = launch_row_sums(st->W, reinterpret_cast<int *>(ws + plan.w_off), st->N, st->K, w_plane_bits(st), (hipStream_t)stream);
                    if (e != hipSuccess)
                        return hip_status(e);
                }
                a.x_row_sums = !need_x ? nullptr : st->x_row_sums ? st->x_row_sums : reinterpret_cast<const int *>(ws + plan.x_off);
                a.w_row_sums = !need_w ? nullptr : st->w_row_sums ? st->w_row_sums : reinterpret_cast<const int *>(ws + plan.w_off);
            } else {
                variant = -1;
                const KernelEntry &want = t->entries[st->variant];
                for (int i = 0; i < st->variant; ++i) {
                    const KernelEntry &o = t->entries[i];
                    if (!(o.flags & kNeedsRowSums) && o.tm == want.tm && o.tn == want.tn && o.wm == want.wm && o.wn == want.wn &&
                        o.wk == want.wk && o.kb == want.kb)
                        variant = i;
                }
                if (variant < 0)
                    return ABQ_ERR_NOT_INITIALIZED;
            }
        }
        e = t->entries[variant].launch(a, (hipStream_t)stream);
    } else {
        if (st->group_size && st->strategy != ABQ_STRATEGY_DECODE)
            return ABQ_ERR_NOT_INITIALIZED; // group scales live on the decode and tiled kernels only
        const KernelTable *tables = st->strategy == ABQ_STRATEGY_BCNT     ? reg.bcnt
                                    : st->strategy == ABQ_STRATEGY_DECODE ? (st->group_size ? reg.decode_grouped : reg.decode)
                                                                          : reg.mfma;
        const KernelTable *t = find_table(tables, c.x_bits, c.w_bits, c.is_signed);
        if (!t || st->variant < 0 || st->variant >= t->count)
            return ABQ_ERR_NOT_INITIALIZED;
        e = t->entries[st->variant].launch(a, (hipStream_t)stream);
    }
    return hip_status(e);
}

size_t abq_planes_bytes(int rows, int k, int bits)
{
    if (rows <= 0 || k <= 0 || bits <= 0 || k % 32)
        return 0;
    return planes_bytes(rows, k, bits);
}

abq_status abq_relayout_planes(const uint32_t *planes, uint32_t *tiled, int rows, int k, int bits, void *stream)
{
    if (!planes || !tiled || rows <= 0 || bits < 1 || bits > 8)
        return ABQ_ERR_INVALID_ARG;
    if (k < 128 || k % 128 != 0)
        return ABQ_ERR_BAD_K;
    return hip_status(launch_relayout_planes(planes, tiled, rows, k, bits, (hipStream_t)stream));
}

size_t abq_fp6_bytes(int rows, int k)
{
    if (rows <= 0 || k <= 0 || k % 128)
        return 0;
    return fp6_bytes(rows, k);
}

int abq_fp6_eligible(int x_bits, int w_bits, int is_signed, int k) { return fp6_eligible(x_bits, w_bits, is_signed, k) ? 1 : 0; }

int abq_prepared_decode_pays(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group_size, int act)
{
    if (M <= 0 || N <= 0 || K < 128 || K % 128 != 0)
        return 0;
    const Registry &reg = registry();
    if (group_size) {
        const KernelTable *t = find_table(reg.decode_tiled_grouped, x_bits, w_bits, is_signed);
        return t && t->count > 0 && (group_size == 128 || group_size == 64) && (!act || N % 32 == 0) &&
                       decode_tiled_grouped_rows(16, act ? 2 : 1, M, K, x_bits, group_size) != 0 &&
                       decode_tiled_grouped_pays(x_bits, w_bits, M, N, K, act, group_size)
                   ? 1
                   : 0;
    }
    const KernelTable *t = find_table(reg.decode_tiled, x_bits, w_bits, is_signed);
    return t && t->count > 0 && !act && decode_tiled_pays(x_bits, w_bits, M, N, K) ? 1 : 0;
}

abq_status abq_relayout_planes_fp6(const uint32_t *planes, uint32_t *fp6, int rows, int k, int bits, int is_signed,
                                   void *stream)
{
    if (!planes || !fp6 || rows <= 0 || bits < 1)
        return ABQ_ERR_INVALID_ARG;
    if (bits > (is_signed ? 5 : 4))
        return ABQ_ERR_UNSUPPORTED;
    if (k < 128 || k % 128 != 0)
        return ABQ_ERR_BAD_K;
    return hip_status(launch_relayout_planes_fp6(planes, fp6, rows, k, bits, is_signed ? 1 : 0, (hipStream_t)stream));
}

abq_status abq_relayout_planes_fp6_folded(const uint32_t *planes, const float *w_zero, int group_size, uint32_t *fp6, int rows, int k,
                                          int bits, int is_signed, int *misfit_dev, void *stream)
{
    if (!planes || !w_zero || !fp6 || rows <= 0 || bits < 1 || group_size < 32 || group_size % 32 != 0)
        return ABQ_ERR_INVALID_ARG;
    if (bits > 4)
        return ABQ_ERR_UNSUPPORTED; // wider codes less their zero points leave the range of the FP6 codes
    if (k < 128 || k % 128 != 0 || k % group_size != 0)
        return ABQ_ERR_BAD_K;
    return hip_status(launch_relayout_planes_fp6(planes, fp6, rows, k, bits, is_signed ? 1 : 0, (hipStream_t)stream, w_zero, group_size,
                                                 misfit_dev));
}

size_t abq_gemm_workspace_bytes(const abq_gemm_state *st)
{
    if (!st || !st->init_success)
        return 0;
    if (st->strategy == ABQ_STRATEGY_FP6)
        return (st->x_layout == ABQ_LAYOUT_FP6 ? 0 : fp6_bytes(st->M, st->K)) +
               (st->w_layout == ABQ_LAYOUT_FP6 ? 0 : fp6_bytes(st->N, st->K));
    // (fp16 activations are quantised inside the decode kernel: nothing is converted for them)
    const int xrec = st->strategy == ABQ_STRATEGY_DECODE_TILED ? decode_tiled_x_bits(st->cfg.x_bits) : st->cfg.x_bits;
    const size_t xb = (st->x_layout == ABQ_LAYOUT_TILED || st->x_layout == ABQ_LAYOUT_F16) ? 0 : planes_bytes(st->M, st->K, xrec);
    const size_t wb = st->w_layout == ABQ_LAYOUT_TILED ? 0 : planes_bytes(st->N, st->K, st->cfg.w_bits);
    // (pairs with an unsigned 8-bit operand on the staged kernel: the row sums of the operands still in planes)
    return xb + wb + (wants_row_sums(st) ? row_sum_plan(st, xb + wb).bytes : 0);
}

static abq_status set_operand_layout_by_rules(abq_gemm_state *st, int x_layout, int w_layout);

} // extern "C"
namespace abq {
bool activations_run_padded(int x_bits, int w_bits, int is_signed, int M, int group_size)
{
    return is_signed && M > 16 && !group_size && x_bits >= 1 && x_bits <= 8 && !one_field(x_bits) && one_field(w_bits) &&
           find_table(registry().tiled, abq_padded_bits(x_bits), w_bits, 1) != nullptr;
}
} // namespace abq
extern "C" {

abq_status abq_gemm_set_operand_layout(abq_gemm_state *st, int x_layout, int w_layout)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    abq_gemm_state next = *st; // the caller's state changes only if the declaration is taken
    abq_status rc = set_operand_layout_by_rules(&next, x_layout, w_layout);
    // Activations of several fields that arrive as planes, against K-tiled weights of one field: exec converts the
    // activations anyway, so they become records of the next single-field width and the state that pair's (the codes'
    // own width kept as value bits, as abq_gemm_set_value_bits would): its LDS-staged kernel instead of the
    // register-staged one of the odd widths (W2A6 at M = 128 on the LLaMA-13B shapes: 1.6 times faster).
    if (rc == ABQ_OK && next.auto_chosen && x_layout == ABQ_LAYOUT_PLANES && w_layout == ABQ_LAYOUT_TILED && !next.act &&
        next.strategy == ABQ_STRATEGY_TILED && next.reserved[2] == 0 && next.reserved[3] == 0 &&
        abq::activations_run_padded(next.cfg.x_bits, next.cfg.w_bits, next.cfg.is_signed, next.M, next.group_size)) {
        abq_gemm_state alt = next;
        alt.reserved[2] = alt.cfg.x_bits;
        alt.reserved[3] = alt.cfg.w_bits;
        alt.cfg.x_bits = abq_padded_bits(alt.cfg.x_bits);
        if (switch_to_tiled(&alt) == ABQ_OK)
            next = alt;
    }
    if (rc == ABQ_OK)
        apply_tuned(&next); // a measured best tile for this shape on these layouts, if the table holds one
    // activation records declared padded are read by the decode kernel on prepared operands only
    if (rc == ABQ_OK && next.x_layout == ABQ_LAYOUT_TILED && padded_x(&next) && next.strategy != ABQ_STRATEGY_DECODE_TILED)
        rc = ABQ_ERR_UNSUPPORTED;
    if (rc == ABQ_OK)
        *st = next;
    return rc;
}

static abq_status set_operand_layout_by_rules(abq_gemm_state *st, int x_layout, int w_layout)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (x_layout < ABQ_LAYOUT_PLANES || x_layout > ABQ_LAYOUT_FP6 || w_layout < ABQ_LAYOUT_PLANES ||
        w_layout > ABQ_LAYOUT_FP6)
        return ABQ_ERR_INVALID_ARG;
    const bool any_fp6 = x_layout == ABQ_LAYOUT_FP6 || w_layout == ABQ_LAYOUT_FP6;
    const bool any_tiled = x_layout == ABQ_LAYOUT_TILED || w_layout == ABQ_LAYOUT_TILED;
    if (any_fp6 && any_tiled)
        return ABQ_ERR_UNSUPPORTED;
    if (any_fp6 && st->strategy != ABQ_STRATEGY_FP6) {
        if (!st->auto_chosen)
            return ABQ_ERR_UNSUPPORTED;
        const abq_status rc = switch_to_fp6(st);
        if (rc != ABQ_OK)
            return rc;
    }
    if (st->strategy == ABQ_STRATEGY_FP6 && any_tiled) {
        if (!st->auto_chosen)
            return ABQ_ERR_UNSUPPORTED;
        const abq_status rc = switch_to_tiled(st);
        if (rc != ABQ_OK)
            return rc;
    }
    // decode-sized M (and up to 128 rows where it pays) with both operands prepared: the decode kernel of that layout
    // (plain and per-channel epilogues)
    if (st->strategy == ABQ_STRATEGY_DECODE_TILED && !decode_tiled_x_ok(st, x_layout)) {
        // activation records of several fields: the prefill kernel reads those
        if (!st->auto_chosen)
            return ABQ_ERR_UNSUPPORTED;
        const abq_status rc = st->group_size ? pick_grouped_tiled(st) : switch_to_tiled(st);
        if (rc != ABQ_OK)
            return rc;
    }
    if (x_layout == ABQ_LAYOUT_TILED && w_layout == ABQ_LAYOUT_TILED && st->auto_chosen && decode_tiled_x_ok(st, x_layout) &&
        decode_tiled_pays(st->cfg.x_bits, st->cfg.w_bits, st->M, st->N, st->K) && !st->group_size &&
        !st->act && st->strategy != ABQ_STRATEGY_DECODE_TILED && switch_to_decode_tiled(st) == ABQ_OK) {
        st->x_layout = x_layout;
        st->w_layout = w_layout;
        return ABQ_OK;
    }
    // the same with group scales attached before the layouts were declared
    if (x_layout == ABQ_LAYOUT_TILED && w_layout == ABQ_LAYOUT_TILED && st->group_size && st->strategy != ABQ_STRATEGY_DECODE_TILED &&
        decode_tiled_grouped_fits(st, st->group_size, st->act) && switch_to_decode_tiled(st) == ABQ_OK) {
        st->variant = 0;
        st->x_layout = x_layout;
        st->w_layout = w_layout;
        return ABQ_OK;
    }
    if (any_tiled && st->strategy != ABQ_STRATEGY_TILED && st->strategy != ABQ_STRATEGY_DECODE_TILED) {
        if (!st->auto_chosen)
            return ABQ_ERR_UNSUPPORTED;
        const abq_status rc = st->group_size ? pick_grouped_tiled(st) : switch_to_tiled(st);
        if (rc != ABQ_OK)
            return rc;
    }
    st->x_layout = x_layout;
    st->w_layout = w_layout;
    return ABQ_OK;
}

abq_status abq_gemm_set_f16_activations(abq_gemm_state *st, const void *x_f16, const float *scale_dev)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (!x_f16 || !scale_dev)
        return ABQ_ERR_INVALID_ARG;
    const abq_tile_config &c = st->cfg;
    const KernelTable *t = find_table(registry().decode_tiled_f16, c.x_bits, c.w_bits, c.is_signed);
    // the quantising instances mirror the first entries of the kernel's table, those of one tile per workgroup; a
    // state whose tile is the library's choice moves to the one its rules pick among them
    if (st->strategy == ABQ_STRATEGY_DECODE_TILED && st->auto_chosen && t && st->variant >= t->count && st->M <= 16 &&
        switch_to_decode_tiled(st, true) != ABQ_OK)
        return ABQ_ERR_UNSUPPORTED;
    if (st->strategy != ABQ_STRATEGY_DECODE_TILED || st->group_size || st->act || st->w_layout != ABQ_LAYOUT_TILED || !t ||
        st->variant < 0 || st->variant >= t->count || (size_t)st->M * st->K * 2 >= (1ull << 32))
        return ABQ_ERR_UNSUPPORTED;
    st->X = static_cast<const uint32_t *>(x_f16);
    st->x_layout = ABQ_LAYOUT_F16;
    st->x_pack_scale = scale_dev;
    return ABQ_OK;
}

abq_status abq_gemm_set_dynamic_f16_activations(abq_gemm_state *st, const void *x_f16, int symmetric)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (!x_f16)
        return ABQ_ERR_INVALID_ARG;
    const abq_tile_config &c = st->cfg;
    const KernelTable *t = find_table(registry().decode_tiled_grouped_dyn, c.x_bits, c.w_bits, c.is_signed);
    // a workgroup quantises all of its rows in registers: 16384 elements (the instance of eight waves; all rows of a
    // call at most 16, which is what the decode kernel takes per workgroup without splitting M)
    if (st->strategy != ABQ_STRATEGY_DECODE_TILED || st->group_size != 128 || st->w_layout != ABQ_LAYOUT_TILED || !t || t->count == 0 ||
        st->variant != 0 || st->M > 16 || (size_t)st->M * st->K > 16384 || (st->x_zero && symmetric))
        return ABQ_ERR_UNSUPPORTED;
    if (!symmetric && !st->w_zero_term && st->x_zero)
        return ABQ_ERR_INVALID_ARG;
    st->X = static_cast<const uint32_t *>(x_f16);
    st->x_layout = ABQ_LAYOUT_F16;
    st->reserved[1] = symmetric ? 1 : 2;
    return ABQ_OK;
}

abq_status abq_gemm_set_workspace(abq_gemm_state *st, void *workspace, size_t bytes)
{
    if (!st || !st->init_success)
        return ABQ_ERR_NOT_INITIALIZED;
    if (!workspace && bytes)
        return ABQ_ERR_INVALID_ARG;
    st->workspace = workspace;
    st->workspace_bytes = bytes;
    // (up to 64 rows, 32 on wide outputs, the conversion launch costs more than the LDS-staged kernel gains over the
    // 16-row tiles on plane operands: W2A8 32 x 4096 x 4096 12.6 against 8.7 us)
    // A state on the decode kernel of prepared operands converts nothing and was weighed against the prefill kernel when
    // it got there: it stays.  A state with group scales moves to the group-scale variants of the prefill kernel (the
    // plain table's variant numbers mean other tiles there).
    const bool pays = st->group_size != 0 || st->M > 64 || (st->M > 32 && st->N >= 8192);
    if (st->strategy != ABQ_STRATEGY_TILED && st->strategy != ABQ_STRATEGY_FP6 && st->strategy != ABQ_STRATEGY_DECODE_TILED &&
        st->auto_chosen && st->M > 16 && pays && workspace && bytes >= abq_gemm_workspace_bytes(st)) {
        const abq_status rc = st->group_size ? pick_grouped_tiled(st) : switch_to_tiled(st);
        if (rc != ABQ_OK)
            return rc;
    }
    // Weights prepared, activations still planes, 17 to 128 rows: the decode kernel of prepared operands where it is
    // estimated ahead of the prefill tile; either kernel has the activations converted into the workspace first, so the
    // estimate is the one of prepared activations (W2A8 32 x 4096 x 4096 from planes: 8.1 against 11.8 us).
    if (st->strategy == ABQ_STRATEGY_TILED && st->auto_chosen && !st->group_size && !st->act && st->M > 16 && workspace &&
        st->x_layout == ABQ_LAYOUT_PLANES && st->w_layout == ABQ_LAYOUT_TILED &&
        decode_tiled_pays(st->cfg.x_bits, st->cfg.w_bits, st->M, st->N, st->K)) {
        abq_gemm_state tmp = *st;
        if (switch_to_decode_tiled(&tmp) == ABQ_OK && decode_tiled_x_ok(&tmp) && bytes >= abq_gemm_workspace_bytes(&tmp))
            *st = tmp;
    }
    apply_tuned(st); // (a tile that converts plane activations can be taken now that there is room for them)
    return ABQ_OK;
}

abq_status abq_gemm_launch(const abq_tile_config *cfg, const uint32_t *X, const uint32_t *W,
                           const void *C, int32_t *D, int bias, int M, int N, int K, void *stream)
{
    if (!cfg)
        return ABQ_ERR_INVALID_ARG;
    abq_gemm_state st;
    abq_status s = abq_gemm_init(cfg, 0, 0, 0, X, W, M, N, K, D, C, bias, ABQ_OUT_I32, &st);
    if (s != ABQ_OK)
        return s;
    return abq_gemm_exec(&st, stream);
}

} // extern "C"
