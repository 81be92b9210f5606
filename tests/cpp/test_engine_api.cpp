// Exercises the C++ face of the library the way the reference's own harness and the FT layers
// use theirs: named Init/Exec globals (engine/test/test_mma/test_mma.h:68-160), launch_pack,
// launchWmmaAnyKernel and ABQGEMMWrapper::gemm.  Results are compared with the CPU oracle
// (oracle/abq_oracle.h) bit for bit.  `--no-gpu` runs only the host-side error paths.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#define ABQ_ALL_COMBOS
#include "common/pack.h"
#include "common/timer.h"
#include "mma_any/aq_bmma_library.h"
#include "mma_any/aq_wmma_library.h"
#include "wmma_any/wmma_any.h"
#include "abq_gemm_wrapper.h"
#include "abq_weight_file.h"
#include "abq_oracle.h"

// reference (tensor-core) tuples, declared here the way a user of the reference would
AQ_DECL_FUN(AqBMMA, 8, 2, true, 1, 48, 512, 8, 24, 128, 8, 8, 128, 4)
AQ_DECL_FUN(AqBMMA, 8, 2, true, 8, 48, 256, 32, 48, 128, 8, 8, 128, 5)
AQ_DECL_FUN(AqBWMMA, 8, 2, false, 8, 48, 256, 32, 48, 128, 8, 8, 128, 5)

static int failures = 0;
#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::printf("CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                    \
        }                                                                  \
    } while (0)
#define HIP_OK(x) CHECK((x) == hipSuccess)

static void host_paths()
{
    int *fake = reinterpret_cast<int *>(0x1000);
    // K constraint (engine/test_any_mma.cu:99): init reports failure, nothing is launched
    AqBMMAOpState st = (*AqBMMA_8x2xtrue_16x16x4096_16x16x512_16x16x64_3_InitFn)(fake, fake, 1, 64, 100, fake, nullptr, false);
    CHECK(!st.initSuccess);
    st = (*AqBMMA_8x2xtrue_16x16x4096_16x16x512_16x16x64_3_InitFn)(fake, fake, 8, 4096, 4096, fake, nullptr, false);
    CHECK(st.initSuccess && st.args.M == 8 && st.args.N == 4096 && st.args.K == 4096);
    CHECK(st.gridDim.x == 256 && st.blockDim.x == 512); // the named 8-wave decode tile
    CHECK(st.native.strategy == ABQ_STRATEGY_DECODE);
    // a reference tuple resolves to the library's choice
    st = (*AqBMMA_8x2xtrue_1x48x512_8x24x128_8x8x128_4_InitFn)(fake, fake, 1, 4096, 4096, fake, nullptr, false);
    CHECK(st.initSuccess && st.native.strategy != ABQ_STRATEGY_AUTO);
    AqBWMMAOpState sw = (*AqBWMMA_8x2xfalse_8x48x256_32x48x128_8x8x128_5_InitFn)(fake, fake, 8, 512, 1024, fake, nullptr, false);
    CHECK(sw.initSuccess);
    // the wrapper refuses bad K and short workspaces before touching the device
    ABQGEMMWrapper wrap(8, 2, true);
    wrap.gemm(1, 64, 100, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, false, nullptr, 0, nullptr);
    wrap.gemm(4, 64, 256, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, false, nullptr, 16, nullptr);
}

struct Case {
    int M, N, K, q, p;
    bool is_signed;
};

static void fill(std::vector<int> &v, int bits, bool is_signed, std::mt19937_64 &rng)
{
    const int lo = is_signed ? -(1 << (bits - 1)) : 0;
    for (auto &e : v)
        e = lo + (int)(rng() % (1u << bits));
}

template <typename InitFn, typename ExecFn, typename State>
static bool run_config(InitFn init_fn, ExecFn exec_fn, const Case &c, int *d_xp, int *d_wp, int *d_out,
                       const std::vector<int> &ref, hipStream_t stream)
{
    HIP_OK(hipMemsetAsync(d_out, 0xff, (size_t)c.M * c.N * 4, stream));
    State state = (*init_fn)(d_xp, d_wp, c.M, c.N, c.K, d_out, nullptr, false);
    if (!state.initSuccess)
        return false;
    (*exec_fn)(state, stream);
    if (hipStreamSynchronize(stream) != hipSuccess || hipGetLastError() != hipSuccess)
        return false;
    std::vector<int> out((size_t)c.M * c.N);
    HIP_OK(hipMemcpy(out.data(), d_out, out.size() * 4, hipMemcpyDeviceToHost));
    return std::memcmp(out.data(), ref.data(), out.size() * 4) == 0;
}

static void gpu_paths()
{
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    std::mt19937_64 rng(7);
    const Case c{ 8, 1000, 1152, 8, 2, true };
    std::vector<int> hx((size_t)c.M * c.K), hw((size_t)c.N * c.K);
    fill(hx, c.q, c.is_signed, rng);
    fill(hw, c.p, c.is_signed, rng);
    const size_t KW = c.K / 32, xw = (size_t)c.q * c.M * KW, ww = (size_t)c.p * c.N * KW;
    int *d_x, *d_w, *d_xp, *d_wp, *d_out;
    HIP_OK(hipMalloc(&d_x, hx.size() * 4));
    HIP_OK(hipMalloc(&d_w, hw.size() * 4));
    HIP_OK(hipMalloc(&d_xp, xw * 4));
    HIP_OK(hipMalloc(&d_wp, ww * 4));
    HIP_OK(hipMalloc(&d_out, (size_t)c.M * c.N * 4));
    HIP_OK(hipMemcpy(d_x, hx.data(), hx.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_w, hw.data(), hw.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(launch_pack(d_w, d_wp, c.N, c.K, c.p, stream));
    HIP_OK(launch_pack(d_x, d_xp, c.M, c.K, c.q, stream));
    HIP_OK(hipStreamSynchronize(stream));

    // packed planes against the oracle's pack, expected GEMM from the oracle's compute_ref
    std::vector<uint32_t> xp(xw), wp(ww), xp_ref(xw), wp_ref(ww);
    HIP_OK(hipMemcpy(xp.data(), d_xp, xw * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(wp.data(), d_wp, ww * 4, hipMemcpyDeviceToHost));
    abq_oracle_pack_i32(hx.data(), xp_ref.data(), c.M, c.K, c.q);
    abq_oracle_pack_i32(hw.data(), wp_ref.data(), c.N, c.K, c.p);
    CHECK(xp == xp_ref && wp == wp_ref);
    std::vector<int> ref((size_t)c.M * c.N);
    abq_oracle_gemm_bitserial(wp_ref.data(), xp_ref.data(), ref.data(), c.M, c.N, c.K, c.p, c.q, c.is_signed);

#define RUN(type, ...)                                                                                        \
    CHECK((run_config<AQ_INIT_FUN(type), AQ_EXEC_FUN(type), AQ_OP_STATE(type)>(                               \
        AQ_NAME_FUN(type, Init, __VA_ARGS__), AQ_NAME_FUN(type, Exec, __VA_ARGS__), c, d_xp, d_wp, d_out, ref, stream)))
    RUN(AqBMMA, 8, 2, true, 1, 16, 4096, 1, 2, 4096, 1, 1, 128, 1);          // VALU popcount
    RUN(AqBMMA, 8, 2, true, 16, 16, 4096, 16, 16, 512, 16, 16, 64, 3);      // decode kernel
    RUN(AqBMMA, 8, 2, true, 16, 16, 4096, 16, 16, 512, 16, 16, 64, 2);      // int8 MFMA 16x16x64
    RUN(AqBMMA, 8, 2, true, 128, 128, 256, 64, 64, 256, 32, 32, 32, 2);     // int8 MFMA 32x32x32
    RUN(AqBWMMA, 8, 2, true, 16, 16, 8192, 16, 16, 512, 16, 16, 64, 3);     // same kernels, wmma names
    RUN(AqBMMA, 8, 2, true, 8, 48, 256, 32, 48, 128, 8, 8, 128, 5);         // FT tile by its reference name
#undef RUN

    {   // first-generation entry point
        HIP_OK(hipMemsetAsync(d_out, 0xff, (size_t)c.M * c.N * 4, stream));
        AnyQuantParams params{ d_xp, d_wp, nullptr, d_out, false, c.M, c.N, c.K };
        hipError_t e = launchWmmaAnyKernel<QuantType<8, 2, true>, ShapeBase<16, 16, 4096>, ShapeBase<16, 16, 512>,
                                           ShapeBase<16, 16, 64>, 3>(params, stream);
        CHECK(e == hipSuccess);
        std::vector<int> out((size_t)c.M * c.N);
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(out.data(), d_out, out.size() * 4, hipMemcpyDeviceToHost));
        CHECK(out == ref);
    }

    {   // FP6 matrix-core tile by its name (W4A4 signed): weights prepared as FP6 records, activations converted
        // per call into the workspace handed to the state
        const Case c6{ 70, 200, 640, 4, 4, true };
        std::vector<int> x6((size_t)c6.M * c6.K), w6((size_t)c6.N * c6.K);
        fill(x6, c6.q, true, rng);
        fill(w6, c6.p, true, rng);
        const size_t kw6 = c6.K / 32, xw6 = (size_t)c6.q * c6.M * kw6, ww6 = (size_t)c6.p * c6.N * kw6;
        std::vector<uint32_t> xp6(xw6), wp6(ww6);
        abq_oracle_pack_i32(x6.data(), xp6.data(), c6.M, c6.K, c6.q);
        abq_oracle_pack_i32(w6.data(), wp6.data(), c6.N, c6.K, c6.p);
        std::vector<int> ref6((size_t)c6.M * c6.N);
        abq_oracle_gemm_bitserial(wp6.data(), xp6.data(), ref6.data(), c6.M, c6.N, c6.K, c6.p, c6.q, true);
        int *d_x6, *d_w6, *d_wf6, *d_o6;
        char *d_ws6;
        HIP_OK(hipMalloc(&d_x6, xw6 * 4));
        HIP_OK(hipMalloc(&d_w6, ww6 * 4));
        HIP_OK(hipMalloc(&d_wf6, abq_fp6_bytes(c6.N, c6.K)));
        HIP_OK(hipMalloc(&d_ws6, abq_fp6_bytes(c6.M, c6.K)));
        HIP_OK(hipMalloc(&d_o6, ref6.size() * 4));
        HIP_OK(hipMemcpy(d_x6, xp6.data(), xw6 * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_w6, wp6.data(), ww6 * 4, hipMemcpyHostToDevice));
        CHECK(abq_fp6_eligible(4, 4, 1, c6.K) == 1 && abq_fp6_eligible(8, 2, 1, c6.K) == 0);
        CHECK(abq_relayout_planes_fp6(reinterpret_cast<uint32_t *>(d_w6), reinterpret_cast<uint32_t *>(d_wf6), c6.N, c6.K,
                                      c6.p, 1, stream) == ABQ_OK);
        AqBMMAOpState st6 = (*AqBMMA_4x4xtrue_128x128x128_64x64x128_32x32x64_5_InitFn)(d_x6, d_wf6, c6.M, c6.N, c6.K, d_o6,
                                                                                        nullptr, false);
        CHECK(st6.initSuccess && st6.native.strategy == ABQ_STRATEGY_FP6);
        CHECK(abq_gemm_set_operand_layout(&st6.native, ABQ_LAYOUT_PLANES, ABQ_LAYOUT_FP6) == ABQ_OK);
        CHECK(abq_gemm_workspace_bytes(&st6.native) == abq_fp6_bytes(c6.M, c6.K));
        CHECK(abq_gemm_exec(&st6.native, stream) == ABQ_ERR_INVALID_ARG); // no workspace yet
        CHECK(abq_gemm_set_workspace(&st6.native, d_ws6, abq_fp6_bytes(c6.M, c6.K)) == ABQ_OK);
        HIP_OK(hipMemsetAsync(d_o6, 0xff, ref6.size() * 4, stream));
        (*AqBMMA_4x4xtrue_128x128x128_64x64x128_32x32x64_5_ExecFn)(st6, stream);
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<int> out6(ref6.size());
        HIP_OK(hipMemcpy(out6.data(), d_o6, out6.size() * 4, hipMemcpyDeviceToHost));
        CHECK(out6 == ref6);
        (void)hipFree(d_x6);
        (void)hipFree(d_w6);
        (void)hipFree(d_wf6);
        (void)hipFree(d_ws6);
        (void)hipFree(d_o6);
    }

    {   // FT wrapper: fp16 activations, static scale, fp16 output scaled by scale_out
        const float in_scale = 21.0f, out_scale = 0.0123f;
        std::vector<uint16_t> ha((size_t)c.M * c.K);
        std::normal_distribution<float> nd(0.f, 2.f);
        std::mt19937 r32(3);
        for (auto &h : ha)
            h = abq_oracle_f32_to_f16(nd(r32));
        _Float16 *d_a, *d_d;
        float *d_scales;
        char *d_ws;
        const size_t ws_bytes = (size_t)c.q * c.M * c.K / 8;
        HIP_OK(hipMalloc(&d_a, ha.size() * 2));
        HIP_OK(hipMalloc(&d_d, (size_t)c.M * c.N * 2));
        HIP_OK(hipMalloc(&d_scales, 8));
        HIP_OK(hipMalloc(&d_ws, ws_bytes));
        HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
        const float scales[2] = { in_scale, out_scale };
        HIP_OK(hipMemcpy(d_scales, scales, 8, hipMemcpyHostToDevice));
        ABQGEMMWrapper wrap(c.q, c.p, c.is_signed);
        wrap.gemm(c.M, c.N, c.K, d_a, d_wp, nullptr, d_d, d_scales, nullptr, d_scales + 1, false, d_ws, ws_bytes, stream);
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<uint16_t> got((size_t)c.M * c.N), want((size_t)c.M * c.N);
        HIP_OK(hipMemcpy(got.data(), d_d, got.size() * 2, hipMemcpyDeviceToHost));
        std::vector<uint32_t> ap(xw);
        abq_oracle_pack_f16(ha.data(), in_scale, ap.data(), c.M, c.K, c.q);
        std::vector<int> acc((size_t)c.M * c.N);
        abq_oracle_gemm_bitserial(wp_ref.data(), ap.data(), acc.data(), c.M, c.N, c.K, c.p, c.q, c.is_signed);
        abq_oracle_epilogue_f16(acc.data(), abq_oracle_f32_to_f16(out_scale), want.data(), (int)acc.size());
        CHECK(got == want);
        HIP_OK(hipFree(d_a));
        HIP_OK(hipFree(d_d));
        HIP_OK(hipFree(d_scales));
        HIP_OK(hipFree(d_ws));
    }

    {   // FT wrapper on a prepared weight: gemm() with unchanged arguments, prefill- and decode-sized, against the
        // CPU oracle (pack_half restated, popcount GEMM, the FT epilogue) bit for bit, and the plane weight beside it
        const int N = 4096, K = 4096, Mmax = 1024;
        std::mt19937 r32(11);
        std::normal_distribution<float> nd(0.f, 2.f);
        std::vector<uint16_t> ha((size_t)Mmax * K);
        for (auto &h : ha)
            h = abq_oracle_f32_to_f16(nd(r32));
        std::vector<uint32_t> wpl((size_t)2 * N * K / 32);
        for (auto &v : wpl)
            v = r32();
        _Float16 *d_a, *d_d0, *d_d1;
        int *d_b0, *d_b1, *d_scratch;
        float *d_scales;
        char *d_ws;
        const size_t ws_bytes = (size_t)8 * Mmax * K / 8, wbytes = wpl.size() * 4;
        CHECK(ABQGEMMWrapper::prepared_weight_bytes(N, K, 2) == wbytes);
        HIP_OK(hipMalloc(&d_a, ha.size() * 2));
        HIP_OK(hipMalloc(&d_d0, (size_t)Mmax * N * 2));
        HIP_OK(hipMalloc(&d_d1, (size_t)Mmax * N * 2));
        HIP_OK(hipMalloc(&d_b0, wbytes));
        HIP_OK(hipMalloc(&d_b1, wbytes));
        HIP_OK(hipMalloc(&d_scratch, wbytes));
        HIP_OK(hipMalloc(&d_scales, 8));
        HIP_OK(hipMalloc(&d_ws, ws_bytes));
        HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_b0, wpl.data(), wbytes, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_b1, wpl.data(), wbytes, hipMemcpyHostToDevice));
        const float in_scale = 21.0f, out_scale = 0.0123f;
        const float scales[2] = { in_scale, out_scale };
        HIP_OK(hipMemcpy(d_scales, scales, 8, hipMemcpyHostToDevice));
        CHECK(!ABQGEMMWrapper::is_prepared(d_b1));
        CHECK(!ABQGEMMWrapper::prepare_weight(d_b1, N, 100, 2, d_scratch, stream)); // K not a multiple of 128
        CHECK(ABQGEMMWrapper::prepare_weight(d_b1, N, K, 2, d_scratch, stream));
        CHECK(ABQGEMMWrapper::is_prepared(d_b1) && !ABQGEMMWrapper::is_prepared(d_b0));
        CHECK(!ABQGEMMWrapper::prepare_weight(d_b1, N, K, 2, d_scratch, stream)); // twice
        ABQGEMMWrapper wrap(8, 2, true);
        // expected: all Mmax rows once (the rows of a smaller call are its first rows)
        std::vector<uint32_t> ap((size_t)8 * Mmax * K / 32);
        abq_oracle_pack_f16(ha.data(), in_scale, ap.data(), Mmax, K, 8);
        std::vector<int> acc((size_t)Mmax * N);
        abq_oracle_gemm_popc(wpl.data(), ap.data(), acc.data(), Mmax, N, K, 2, 8, 1, 0);
        std::vector<uint16_t> want((size_t)Mmax * N);
        abq_oracle_epilogue_f16(acc.data(), abq_oracle_f32_to_f16(out_scale), want.data(), (int)acc.size());
        for (int M : { 1024, 300, 16, 8, 4, 2, 1 }) {
            for (int prepared = 0; prepared < 2; ++prepared) {
                _Float16 *d_d = prepared ? d_d1 : d_d0;
                HIP_OK(hipMemsetAsync(d_d, 0xff, (size_t)M * N * 2, stream));
                wrap.gemm(M, N, K, d_a, prepared ? d_b1 : d_b0, nullptr, d_d, d_scales, nullptr, d_scales + 1, false, d_ws, ws_bytes, stream);
                HIP_OK(hipStreamSynchronize(stream));
                std::vector<uint16_t> got((size_t)M * N);
                HIP_OK(hipMemcpy(got.data(), d_d, got.size() * 2, hipMemcpyDeviceToHost));
                CHECK(std::equal(got.begin(), got.end(), want.begin()));
            }
        }
        // the records are where prepare_weight left them; refilled behind the table's back they are not
        CHECK(ABQGEMMWrapper::verify_prepared(d_b1, stream));
        {
            std::vector<uint32_t> keep(16), junk(16, 0x12345678u);
            HIP_OK(hipMemcpy(keep.data(), d_b1, 64, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(d_b1, junk.data(), 64, hipMemcpyHostToDevice));
            CHECK(!ABQGEMMWrapper::verify_prepared(d_b1, stream));
            HIP_OK(hipMemcpy(d_b1, keep.data(), 64, hipMemcpyHostToDevice));
            CHECK(ABQGEMMWrapper::verify_prepared(d_b1, stream));
            CHECK(!ABQGEMMWrapper::verify_prepared(d_b0, stream)); // never prepared
        }
        // gemm_scaled reads planes: a prepared weight is refused (D stays as it was)
        HIP_OK(hipMemset(d_d1, 0xff, 64));
        wrap.gemm_scaled(1, N, K, reinterpret_cast<const int *>(d_ws), d_b1, d_d1, d_scales, d_scales, stream);
        HIP_OK(hipStreamSynchronize(stream));
        {
            uint16_t first = 0;
            HIP_OK(hipMemcpy(&first, d_d1, 2, hipMemcpyDeviceToHost));
            CHECK(first == 0xffff);
        }
        // a prepared weight is checked against the shape it was prepared for: D stays as it was
        HIP_OK(hipMemset(d_d1, 0xff, 64));
        wrap.gemm(1, N / 2, K, d_a, d_b1, nullptr, d_d1, d_scales, nullptr, d_scales + 1, false, d_ws, ws_bytes, stream);
        HIP_OK(hipStreamSynchronize(stream));
        uint16_t first = 0;
        HIP_OK(hipMemcpy(&first, d_d1, 2, hipMemcpyDeviceToHost));
        CHECK(first == 0xffff);
        ABQGEMMWrapper::release_weight(d_b1);
        CHECK(!ABQGEMMWrapper::is_prepared(d_b1));
        HIP_OK(hipFree(d_a));
        HIP_OK(hipFree(d_d0));
        HIP_OK(hipFree(d_d1));
        HIP_OK(hipFree(d_b0));
        HIP_OK(hipFree(d_b1));
        HIP_OK(hipFree(d_scratch));
        HIP_OK(hipFree(d_scales));
        HIP_OK(hipFree(d_ws));
    }

    {   // FT wrapper, W4A4 with the weight also registered as FP6 records: prefill-sized gemm() runs the FP6 matrix
        // cores (activations packed as FP6 records), decode-sized calls keep the other routes; both against the oracle
        const int N = 320, K = 640, Mmax = 300;
        std::mt19937 r32(23);
        std::normal_distribution<float> nd(0.f, 2.f);
        std::vector<uint16_t> ha((size_t)Mmax * K);
        for (auto &h : ha)
            h = abq_oracle_f32_to_f16(nd(r32));
        std::vector<uint32_t> wpl((size_t)4 * N * K / 32);
        for (auto &v : wpl)
            v = r32();
        _Float16 *d_a, *d_d;
        int *d_b, *d_rec, *d_scratch;
        float *d_scales;
        char *d_ws;
        const size_t ws_bytes = (size_t)Mmax * K, wbytes = wpl.size() * 4; // 0.75 M K needed for FP6 records
        HIP_OK(hipMalloc(&d_a, ha.size() * 2));
        HIP_OK(hipMalloc(&d_d, (size_t)Mmax * N * 2));
        HIP_OK(hipMalloc(&d_b, wbytes));
        HIP_OK(hipMalloc(&d_scratch, wbytes));
        HIP_OK(hipMalloc(&d_rec, ABQGEMMWrapper::fp6_weight_bytes(N, K)));
        HIP_OK(hipMalloc(&d_scales, 8));
        HIP_OK(hipMalloc(&d_ws, ws_bytes));
        HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_b, wpl.data(), wbytes, hipMemcpyHostToDevice));
        const float in_scale = 1.7f, out_scale = 0.031f;
        const float scales[2] = { in_scale, out_scale };
        HIP_OK(hipMemcpy(d_scales, scales, 8, hipMemcpyHostToDevice));
        CHECK(!ABQGEMMWrapper::prepare_weight_fp6(d_b, N, K, 6, true, d_rec, stream)); // too wide for FP6 codes
        CHECK(ABQGEMMWrapper::prepare_weight_fp6(d_b, N, K, 4, true, d_rec, stream));
        CHECK(ABQGEMMWrapper::prepare_weight(d_b, N, K, 4, d_scratch, stream));
        CHECK(!ABQGEMMWrapper::prepare_weight_fp6(d_b, N, K, 4, true, d_rec, stream)); // the planes are gone
        std::vector<uint32_t> ap((size_t)4 * Mmax * K / 32);
        abq_oracle_pack_f16(ha.data(), in_scale, ap.data(), Mmax, K, 4);
        std::vector<int> acc((size_t)Mmax * N);
        abq_oracle_gemm_popc(wpl.data(), ap.data(), acc.data(), Mmax, N, K, 4, 4, 1, 0);
        std::vector<uint16_t> want((size_t)Mmax * N);
        abq_oracle_epilogue_f16(acc.data(), abq_oracle_f32_to_f16(out_scale), want.data(), (int)acc.size());
        ABQGEMMWrapper wrap(4, 4, true);
        for (int M : { 300, 128, 16, 1 }) {
            HIP_OK(hipMemsetAsync(d_d, 0xff, (size_t)M * N * 2, stream));
            wrap.gemm(M, N, K, d_a, d_b, nullptr, d_d, d_scales, nullptr, d_scales + 1, false, d_ws, ws_bytes, stream);
            HIP_OK(hipStreamSynchronize(stream));
            std::vector<uint16_t> got((size_t)M * N);
            HIP_OK(hipMemcpy(got.data(), d_d, got.size() * 2, hipMemcpyDeviceToHost));
            CHECK(std::equal(got.begin(), got.end(), want.begin()));
        }
        ABQGEMMWrapper::release_weight(d_b);
        HIP_OK(hipFree(d_a));
        HIP_OK(hipFree(d_d));
        HIP_OK(hipFree(d_b));
        HIP_OK(hipFree(d_scratch));
        HIP_OK(hipFree(d_rec));
        HIP_OK(hipFree(d_scales));
        HIP_OK(hipFree(d_ws));
    }

    // FT wrapper, dynamic path: per-token int8 activations, weights with group scales and zero points; expected
    // values from a double-precision loop over the dequantised operands.  2-bit weights (prefill- and decode-sized
    // calls), and 3-bit weights (the reference's bit-balanced 2-bit quantiser writes three planes): at decode sizes as
    // padded records on the prepared-operand decode kernel of the 4-bit width, as planes on the plane-operand one,
    // above that on the prefill kernel of the padded pair (padded records, which then are the only copy handed over)
    // or of the 3-bit records.
    auto dynamic_case = [&](const int WB, const int M, const bool padded_records, const bool keep_planes, const bool folded_records = false) {
        const int N = 192, K = 512, G = 128, groups = K / G;
        std::mt19937 r32(5 + WB + M);
        std::normal_distribution<float> nd(0.f, 1.5f);
        std::uniform_real_distribution<float> ud(0.002f, 0.02f);
        std::vector<uint16_t> ha((size_t)M * K);
        for (auto &h : ha)
            h = abq_oracle_f32_to_f16(nd(r32));
        std::vector<int> wq((size_t)N * K);
        for (auto &v : wq)
            v = (int)(r32() % (1u << WB)) - (1 << (WB - 1));
        std::vector<float> wscale((size_t)N * groups), wzero((size_t)N * groups);
        for (auto &v : wscale)
            v = ud(r32);
        for (auto &v : wzero)
            v = (float)((int)(r32() % (1u << WB)) - (1 << (WB - 1)));
        std::vector<uint32_t> wpl((size_t)WB * N * K / 32);
        abq_oracle_pack_i32(wq.data(), wpl.data(), N, K, WB);
        _Float16 *d_a, *d_d;
        uint32_t *d_wpl, *d_wt, *d_wpad, *d_wfold;
        int *d_misfit;
        float *d_wscale, *d_wzero, *d_term;
        char *d_ws;
        ABQGEMMWrapper wrap(8, WB, true);
        const size_t ws_bytes = wrap.dynamic_workspace_bytes(M, K, G);
        HIP_OK(hipMalloc(&d_a, ha.size() * 2));
        HIP_OK(hipMalloc(&d_d, (size_t)M * N * 2));
        HIP_OK(hipMalloc(&d_wpl, wpl.size() * 4));
        HIP_OK(hipMalloc(&d_wt, wpl.size() * 4));
        HIP_OK(hipMalloc(&d_wpad, abq_planes_bytes(N, K, abq_padded_bits(WB))));
        HIP_OK(hipMalloc(&d_wfold, abq_planes_bytes(N, K, abq_folded_bits(WB))));
        HIP_OK(hipMalloc(&d_misfit, sizeof(int)));
        HIP_OK(hipMemset(d_misfit, 0, sizeof(int)));
        HIP_OK(hipMalloc(&d_wscale, wscale.size() * 4));
        HIP_OK(hipMalloc(&d_wzero, wzero.size() * 4));
        HIP_OK(hipMalloc(&d_term, N * 4));
        HIP_OK(hipMalloc(&d_ws, ws_bytes));
        HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_wpl, wpl.data(), wpl.size() * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_wscale, wscale.data(), wscale.size() * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_wzero, wzero.data(), wzero.size() * 4, hipMemcpyHostToDevice));
        CHECK(abq_relayout_planes(d_wpl, d_wt, N, K, WB, stream) == ABQ_OK);
        CHECK(abq_relayout_planes_padded(d_wpl, d_wpad, N, K, WB, 1, stream) == ABQ_OK);
        CHECK(abq_weight_zero_term(d_wpl, N, K, WB, 1, d_wscale, d_wzero, G, d_term, stream) == ABQ_OK);
        CHECK(abq_relayout_planes_folded(d_wpl, d_wzero, G, d_wfold, N, K, WB, 1, d_misfit, stream) == ABQ_OK);
        int misfit = 1;
        HIP_OK(hipMemcpy(&misfit, d_misfit, sizeof(int), hipMemcpyDeviceToHost));
        CHECK(misfit == 0);
        const ABQGroupedWeight weight = { padded_records ? nullptr : reinterpret_cast<const int *>(d_wt), d_wscale, d_wzero, d_term, G,
                                          keep_planes ? reinterpret_cast<const int *>(d_wpl) : nullptr, nullptr,
                                          padded_records ? reinterpret_cast<const int *>(d_wpad) : nullptr,
                                          folded_records ? reinterpret_cast<const int *>(d_wfold) : nullptr };
        for (int symmetric = 1; symmetric >= 0; --symmetric) {
            wrap.gemm_dynamic(M, N, K, d_a, weight, d_d, symmetric != 0, d_ws, ws_bytes, stream);
            HIP_OK(hipStreamSynchronize(stream));
            std::vector<uint16_t> got((size_t)M * N);
            HIP_OK(hipMemcpy(got.data(), d_d, got.size() * 2, hipMemcpyDeviceToHost));
            double worst = 0, ref_sq = 0;
            std::vector<double> want((size_t)M * N);
            for (int m = 0; m < M; ++m) {
                // the per-token quantiser in float, as the kernel defines it
                float mx = -INFINITY, mn = INFINITY;
                for (int k = 0; k < K; ++k) {
                    const float f = abq_oracle_f16_to_f32(ha[(size_t)m * K + k]);
                    mx = std::fmax(mx, f);
                    mn = std::fmin(mn, f);
                }
                float scale, zp = 0.f;
                if (symmetric) {
                    scale = std::fmin(std::fmax(std::fmax(std::fabs(mx), std::fabs(mn)) / 127.f, 1e-5f), 1e4f);
                } else {
                    scale = std::fmin(std::fmax((mx - mn) / 255.f, 1e-5f), 1e4f);
                    zp = std::nearbyint(std::fmin(std::fmax(-mn / scale, -1e4f), 1e4f));
                }
                std::vector<double> xd(K);
                for (int k = 0; k < K; ++k) {
                    const float f = abq_oracle_f16_to_f32(ha[(size_t)m * K + k]);
                    float code = std::nearbyint(f / scale) + zp;
                    code = symmetric ? std::fmin(std::fmax(code, -128.f), 127.f) : std::fmin(std::fmax(code, 0.f), 255.f);
                    xd[k] = ((double)code - zp) * scale;
                }
                for (int n = 0; n < N; ++n) {
                    double acc = 0;
                    for (int k = 0; k < K; ++k)
                        acc += xd[k] * ((double)wq[(size_t)n * K + k] - wzero[(size_t)n * groups + k / G]) *
                               wscale[(size_t)n * groups + k / G];
                    want[(size_t)m * N + n] = acc;
                    ref_sq += acc * acc;
                }
            }
            const double rms = std::sqrt(ref_sq / want.size());
            for (size_t i = 0; i < want.size(); ++i) {
                const double err = std::fabs((double)abq_oracle_f16_to_f32(got[i]) - want[i]);
                worst = std::fmax(worst, err / (std::fabs(want[i]) + rms));
            }
            CHECK(worst <= 1e-2); // the 1e-2 relative tolerance of the fp16 dequantised output
        }
        HIP_OK(hipFree(d_a));
        HIP_OK(hipFree(d_d));
        HIP_OK(hipFree(d_wpl));
        HIP_OK(hipFree(d_wt));
        HIP_OK(hipFree(d_wpad));
        HIP_OK(hipFree(d_wfold));
        HIP_OK(hipFree(d_misfit));
        HIP_OK(hipFree(d_wscale));
        HIP_OK(hipFree(d_wzero));
        HIP_OK(hipFree(d_term));
        HIP_OK(hipFree(d_ws));
    };
    dynamic_case(2, 40, false, false);
    dynamic_case(2, 1, false, false);
    dynamic_case(3, 40, true, false);  // blocks of 16 rows on the 4-bit decode kernel (or the prefill kernel on the 3-bit records)
    dynamic_case(3, 1, true, false);   // one launch: the 4-bit decode kernel quantises the row itself
    dynamic_case(3, 8, true, false);   // quantiser + the 4-bit decode kernel on the padded records
    dynamic_case(3, 8, false, true);   // no padded records: the decode kernel on plane operands
    dynamic_case(5, 4, true, false);   // 5-bit weights as 8-bit records
    dynamic_case(3, 300, true, false); // prefill on the padded records: the 4-bit pair's LDS-staged kernel
    dynamic_case(3, 300, false, false); // ... and on the 3-bit records
    dynamic_case(6, 130, true, false); // 6-bit weights as 8-bit records, prefill
    dynamic_case(2, 300, false, false, true); // prefill on records with the zero points folded in (4-bit records of 2-bit weights)
    dynamic_case(3, 300, true, false, true);  // ... of 3-bit weights
    dynamic_case(2, 8, false, false, true);   // decode-sized: the weights' own records
    dynamic_case(3, 8, false, false, true);   // 3-bit weights: the folded records at every size (decode kernel, two launches)
    dynamic_case(3, 1, false, false, true);   // ... one launch
    dynamic_case(3, 40, false, false, true);

    for (const int WB : { 4, 3 })
    for (const int M : { 24, 3 }) {
        // weight file -> device weight -> dynamic GEMM: the file round-trips, and the GEMM on the loaded
        // weight equals a double-precision loop over the blob's own dequantised codes (3-bit weights: the loaded
        // weight carries padded records, which the calls of every size run on)
        const int N = 160, K = 384, G = 64, groups = K / G;
        std::mt19937 r32(11 + WB + M);
        std::normal_distribution<float> nd(0.f, 0.05f), xd_(0.f, 1.f);
        std::vector<float> wf((size_t)N * K);
        for (auto &v : wf)
            v = nd(r32);
        ABQWeightBlob blob, back;
        std::string err;
        CHECK(abq_quantize_weights(wf.data(), N, K, WB, false, G, &blob, &err));
        const std::string path = "/tmp/abq_test_weight.abqw";
        CHECK(abq_weight_file_write(path, blob, &err));
        CHECK(abq_weight_file_read(path, &back, &err));
        CHECK(back.planes == blob.planes && back.scale == blob.scale && back.zero == blob.zero &&
              std::memcmp(&back.info, &blob.info, sizeof(blob.info)) == 0);
        CHECK(!abq_weight_file_read("/tmp/abq_no_such_file.abqw", &back, &err));
        std::remove(path.c_str());
        ABQDeviceWeight dw;
        CHECK(dw.load(blob, stream, &err));
        // (3-bit weights: padded records, or, their zero points being whole numbers, folded ones of the same width)
        CHECK((dw.grouped().records_padded != nullptr || dw.grouped().records_folded != nullptr) == (WB == 3 || dw.grouped().records_folded != nullptr));
        CHECK(WB != 3 || dw.grouped().records_folded != nullptr);
        std::vector<int> codes((size_t)N * K);
        abq_oracle_unpack(blob.planes.data(), codes.data(), N, K, WB, 1);
        std::vector<uint16_t> ha((size_t)M * K);
        for (auto &h : ha)
            h = abq_oracle_f32_to_f16(xd_(r32));
        ABQGEMMWrapper wrap(8, WB, true);
        const size_t ws_bytes = wrap.dynamic_workspace_bytes(M, K, G);
        _Float16 *d_a, *d_d;
        char *d_ws;
        HIP_OK(hipMalloc(&d_a, ha.size() * 2));
        HIP_OK(hipMalloc(&d_d, (size_t)M * N * 2));
        HIP_OK(hipMalloc(&d_ws, ws_bytes));
        HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
        wrap.gemm_dynamic(M, N, K, d_a, dw.grouped(), d_d, true, d_ws, ws_bytes, stream);
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<uint16_t> got((size_t)M * N);
        HIP_OK(hipMemcpy(got.data(), d_d, got.size() * 2, hipMemcpyDeviceToHost));
        double worst = 0, ref_sq = 0;
        std::vector<double> want((size_t)M * N);
        for (int m = 0; m < M; ++m) {
            float amax = 0.f;
            for (int k = 0; k < K; ++k)
                amax = std::fmax(amax, std::fabs(abq_oracle_f16_to_f32(ha[(size_t)m * K + k])));
            const float scale = std::fmin(std::fmax(amax / 127.f, 1e-5f), 1e4f);
            for (int n = 0; n < N; ++n) {
                double acc = 0;
                for (int k = 0; k < K; ++k) {
                    const float code = std::fmin(std::fmax(std::nearbyint(abq_oracle_f16_to_f32(ha[(size_t)m * K + k]) / scale), -128.f), 127.f);
                    acc += (double)code * scale * ((double)codes[(size_t)n * K + k] - blob.zero[(size_t)n * groups + k / G]) *
                           blob.scale[(size_t)n * groups + k / G];
                }
                want[(size_t)m * N + n] = acc;
                ref_sq += acc * acc;
            }
        }
        const double rms = std::sqrt(ref_sq / want.size());
        for (size_t i = 0; i < want.size(); ++i)
            worst = std::fmax(worst, std::fabs((double)abq_oracle_f16_to_f32(got[i]) - want[i]) / (std::fabs(want[i]) + rms));
        CHECK(worst <= 1e-2);
        HIP_OK(hipFree(d_a));
        HIP_OK(hipFree(d_d));
        HIP_OK(hipFree(d_ws));
    }

    {   // W4A4 with groups of 128: a loaded weight also carries FP6 records, and calls of more than 256 rows run
        // on the FP6 matrix cores (below, the int8 route's small tiles are ahead and both weights take the same
        // kernel); same output as the int8 route (the integer tiles are exact on both and are folded in the same order)
        const int N = 192, K = 512, G = 128;
        std::mt19937 r32(23);
        std::normal_distribution<float> nd(0.f, 0.05f), xd_(0.f, 1.f);
        std::vector<float> wf((size_t)N * K);
        for (auto &v : wf)
            v = nd(r32);
        ABQWeightBlob blob;
        std::string err;
        CHECK(abq_quantize_weights(wf.data(), N, K, 4, false, G, &blob, &err));
        ABQDeviceWeight dw;
        CHECK(dw.load(blob, stream, &err));
        ABQGroupedWeight with_fp6 = dw.grouped(), without = dw.grouped();
        // (the zero points of the quantiser are whole numbers: the FP6 records hold code - zero point)
        CHECK(with_fp6.records_fp6 == nullptr && with_fp6.records_fp6_folded != nullptr);
        without.records_fp6 = without.records_fp6_folded = nullptr;
        without.records_folded = nullptr; // (W4A4 has no pair for 8-bit folded records anyway)
        CHECK(abq_preferred_weight_layout(4, 4, 1, 300, N, K, G) == ABQ_LAYOUT_FP6 && abq_preferred_weight_layout(4, 4, 1, 40, N, K, G) == ABQ_LAYOUT_TILED);
        for (const int M : { 300, 40 }) {
        std::vector<uint16_t> ha((size_t)M * K);
        for (auto &h : ha)
            h = abq_oracle_f32_to_f16(xd_(r32));
        ABQGEMMWrapper wrap(4, 4, true);
        const size_t ws_bytes = wrap.dynamic_workspace_bytes(M, K, G);
        CHECK(wrap.activation_bytes(M, K) >= (size_t)M * K * 6 / 8);
        _Float16 *d_a, *d_d;
        char *d_ws;
        HIP_OK(hipMalloc(&d_a, ha.size() * 2));
        HIP_OK(hipMalloc(&d_d, (size_t)M * N * 2));
        HIP_OK(hipMalloc(&d_ws, ws_bytes));
        HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
        std::vector<uint16_t> got_fp6((size_t)M * N), got_int8((size_t)M * N);
        for (int symmetric = 1; symmetric >= 0; --symmetric) {
            HIP_OK(hipMemset(d_d, 0, (size_t)M * N * 2));
            wrap.gemm_dynamic(M, N, K, d_a, with_fp6, d_d, symmetric != 0, d_ws, ws_bytes, stream);
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipMemcpy(got_fp6.data(), d_d, got_fp6.size() * 2, hipMemcpyDeviceToHost));
            HIP_OK(hipMemset(d_d, 0, (size_t)M * N * 2));
            wrap.gemm_dynamic(M, N, K, d_a, without, d_d, symmetric != 0, d_ws, ws_bytes, stream);
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipMemcpy(got_int8.data(), d_d, got_int8.size() * 2, hipMemcpyDeviceToHost));
            size_t nonzero = 0, differ = 0;
            double worst = 0, sq = 0;
            for (size_t i = 0; i < got_int8.size(); ++i) {
                const double b = abq_oracle_f16_to_f32(got_int8[i]);
                sq += b * b;
            }
            const double rms = std::sqrt(sq / (double)got_int8.size());
            for (size_t i = 0; i < got_fp6.size(); ++i) {
                nonzero += got_fp6[i] != 0;
                differ += got_fp6[i] != got_int8[i];
                const double a = abq_oracle_f16_to_f32(got_fp6[i]), b = abq_oracle_f16_to_f32(got_int8[i]);
                // (entries that cancel to nearly nothing carry the rounding of terms of the size of the matrix's RMS)
                worst = std::fmax(worst, std::fabs(a - b) / (std::fabs(b) + 0.5 * rms));
            }
            CHECK(nonzero > got_fp6.size() / 2);
            CHECK(worst <= 2e-3); // one fp16 unit at most: the zero-point terms are summed in a different association
            if (worst > 2e-3)
                std::printf("  M = %d symmetric = %d: worst %.3g, rms %.3g, %zu of %zu differ\n", M, symmetric, worst, rms, differ, got_fp6.size());
        }
        HIP_OK(hipFree(d_a));
        HIP_OK(hipFree(d_d));
        HIP_OK(hipFree(d_ws));
        }
    }

    {   // gate / up pair through the weight-blob interleave and the fused SiLU-gate epilogue, decode- and
        // prefill-sized M, against silu(gate GEMM) * (up GEMM) run as two separate dynamic GEMMs
        const int I = 96, K = 256, G = 128;
        std::mt19937 r32(17);
        std::normal_distribution<float> nd(0.f, 0.05f), xd_(0.f, 1.f);
        std::vector<float> wg((size_t)I * K), wu((size_t)I * K);
        for (auto &v : wg)
            v = nd(r32);
        for (auto &v : wu)
            v = nd(r32);
        ABQWeightBlob bg, bu, bcat;
        std::string err;
        CHECK(abq_quantize_weights(wg.data(), I, K, 2, false, G, &bg, &err));
        CHECK(abq_quantize_weights(wu.data(), I, K, 2, false, G, &bu, &err));
        CHECK(abq_weight_blob_interleave_gate_up(bg, bu, &bcat, &err));
        CHECK(bcat.info.n == 2 * I && bcat.planes.size() == 2 * bg.planes.size());
        ABQDeviceWeight dg, du, dcat;
        CHECK(dg.load(bg, stream, &err) && du.load(bu, stream, &err) && dcat.load(bcat, stream, &err));
        ABQGEMMWrapper wrap(8, 2, true);
        for (int M : { 3, 70 }) {
            std::vector<uint16_t> ha((size_t)M * K);
            for (auto &h : ha)
                h = abq_oracle_f32_to_f16(xd_(r32));
            const size_t ws_bytes = wrap.dynamic_workspace_bytes(M, K, G);
            _Float16 *d_a, *d_g, *d_u, *d_f;
            char *d_ws;
            HIP_OK(hipMalloc(&d_a, ha.size() * 2));
            HIP_OK(hipMalloc(&d_g, (size_t)M * I * 2));
            HIP_OK(hipMalloc(&d_u, (size_t)M * I * 2));
            HIP_OK(hipMalloc(&d_f, (size_t)M * I * 2));
            HIP_OK(hipMalloc(&d_ws, ws_bytes));
            HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
            wrap.gemm_dynamic(M, I, K, d_a, dg.grouped(), d_g, false, d_ws, ws_bytes, stream);
            wrap.gemm_dynamic(M, I, K, d_a, du.grouped(), d_u, false, d_ws, ws_bytes, stream);
            wrap.gemm_dynamic(M, 2 * I, K, d_a, dcat.grouped(), d_f, false, d_ws, ws_bytes, stream, true);
            HIP_OK(hipStreamSynchronize(stream));
            std::vector<uint16_t> hg((size_t)M * I), hu((size_t)M * I), hf((size_t)M * I);
            HIP_OK(hipMemcpy(hg.data(), d_g, hg.size() * 2, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(hu.data(), d_u, hu.size() * 2, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(hf.data(), d_f, hf.size() * 2, hipMemcpyDeviceToHost));
            double worst = 0, rms = 0;
            std::vector<double> want(hf.size());
            for (size_t i = 0; i < hf.size(); ++i) {
                const double gv = abq_oracle_f16_to_f32(hg[i]), uv = abq_oracle_f16_to_f32(hu[i]);
                want[i] = gv / (1.0 + std::exp(-gv)) * uv;
                rms += want[i] * want[i];
            }
            rms = std::sqrt(rms / want.size());
            for (size_t i = 0; i < hf.size(); ++i)
                worst = std::fmax(worst, std::fabs((double)abq_oracle_f16_to_f32(hf[i]) - want[i]) / (std::fabs(want[i]) + rms));
            CHECK(worst <= 1e-2); // the separate GEMMs round gate and up to fp16 first: well inside the tolerance
            HIP_OK(hipFree(d_a));
            HIP_OK(hipFree(d_g));
            HIP_OK(hipFree(d_u));
            HIP_OK(hipFree(d_f));
            HIP_OK(hipFree(d_ws));
        }
    }

    {   // the smallest dynamic calls on prepared weights with groups of 128: one launch that quantises the rows
        // itself; the workspace stays untouched and the output equals, bit for bit, quantise + GEMM called
        // through the C interface
        const int N = 320, K = 1024, G = 128;
        std::mt19937 r32(29);
        std::normal_distribution<float> nd(0.f, 0.05f), xd_(0.3f, 1.f);
        std::vector<float> wf((size_t)N * K);
        for (auto &v : wf)
            v = nd(r32);
        ABQWeightBlob blob;
        std::string err;
        CHECK(abq_quantize_weights(wf.data(), N, K, 2, false, G, &blob, &err));
        ABQDeviceWeight dw;
        CHECK(dw.load(blob, stream, &err));
        const ABQGroupedWeight W = dw.grouped();
        ABQGEMMWrapper wrap(8, 2, true);
        for (int M : { 1, 5, 16 })
            for (int symmetric = 0; symmetric < 2; ++symmetric) {
                std::vector<uint16_t> ha((size_t)M * K);
                for (auto &h : ha)
                    h = abq_oracle_f32_to_f16(xd_(r32));
                const size_t ws_bytes = wrap.dynamic_workspace_bytes(M, K, G);
                _Float16 *d_a, *d_d, *d_e;
                char *d_ws, *d_ws2;
                HIP_OK(hipMalloc(&d_a, ha.size() * 2));
                HIP_OK(hipMalloc(&d_d, (size_t)M * N * 2));
                HIP_OK(hipMalloc(&d_e, (size_t)M * N * 2));
                HIP_OK(hipMalloc(&d_ws, ws_bytes));
                HIP_OK(hipMalloc(&d_ws2, ws_bytes));
                HIP_OK(hipMemcpy(d_a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
                HIP_OK(hipMemset(d_ws, 0xAB, ws_bytes));
                HIP_OK(hipMemset(d_d, 0, (size_t)M * N * 2));
                CHECK(abq_prepared_decode_pays(8, 2, 1, M, N, K, G, ABQ_ACT_NONE) == 1);
                wrap.gemm_dynamic(M, N, K, d_a, W, d_d, symmetric != 0, d_ws, ws_bytes, stream);
                HIP_OK(hipStreamSynchronize(stream));
                std::vector<unsigned char> hws(ws_bytes);
                HIP_OK(hipMemcpy(hws.data(), d_ws, ws_bytes, hipMemcpyDeviceToHost));
                bool untouched = true;
                for (unsigned char b : hws)
                    untouched = untouched && b == 0xAB;
                CHECK(untouched);
                // the same call as two launches
                const size_t planes_bytes = ((size_t)M * K + 255) / 256 * 256;
                uint32_t *planes = reinterpret_cast<uint32_t *>(d_ws2);
                float *x_scale = reinterpret_cast<float *>(d_ws2 + planes_bytes);
                float *x_zero = x_scale + M;
                int32_t *sums = reinterpret_cast<int32_t *>(x_zero + M);
                CHECK(planes_bytes + (size_t)M * 8 + (size_t)M * (K / G) * 4 <= ws_bytes);
                CHECK(abq_quant_pack_f16(d_a, M, K, 8, symmetric, ABQ_LAYOUT_TILED, planes, x_scale, x_zero, sums, G,
                                         stream) == ABQ_OK);
                abq_gemm_state st;
                CHECK(abq_gemm_init(nullptr, 8, 2, 1, planes, reinterpret_cast<const uint32_t *>(W.planes_tiled), M, N,
                                    K, d_e, nullptr, 0, ABQ_OUT_F16_SCALED, &st) == ABQ_OK);
                CHECK(abq_gemm_set_operand_layout(&st, ABQ_LAYOUT_TILED, ABQ_LAYOUT_TILED) == ABQ_OK);
                CHECK(abq_gemm_set_scales(&st, x_scale, W.scale, G) == ABQ_OK);
                CHECK(abq_gemm_set_zero_points(&st, symmetric ? nullptr : x_zero, W.zero, sums,
                                               symmetric ? nullptr : W.zero_term) == ABQ_OK);
                CHECK(abq_gemm_exec(&st, stream) == ABQ_OK);
                HIP_OK(hipStreamSynchronize(stream));
                std::vector<uint16_t> got((size_t)M * N), want((size_t)M * N);
                HIP_OK(hipMemcpy(got.data(), d_d, got.size() * 2, hipMemcpyDeviceToHost));
                HIP_OK(hipMemcpy(want.data(), d_e, want.size() * 2, hipMemcpyDeviceToHost));
                bool nonzero = false;
                for (uint16_t h : want)
                    nonzero = nonzero || (h & 0x7fff);
                CHECK(nonzero);
                CHECK(got == want);
                HIP_OK(hipFree(d_a));
                HIP_OK(hipFree(d_d));
                HIP_OK(hipFree(d_e));
                HIP_OK(hipFree(d_ws));
                HIP_OK(hipFree(d_ws2));
            }
    }

    {   // timer interface
        CudaTimer t(stream);
        t.start();
        t.stop();
        CHECK(t.elapsed_msecs() >= 0.f);
    }
    HIP_OK(hipFree(d_x));
    HIP_OK(hipFree(d_w));
    HIP_OK(hipFree(d_xp));
    HIP_OK(hipFree(d_wp));
    HIP_OK(hipFree(d_out));
    HIP_OK(hipStreamDestroy(stream));
}

int main(int argc, char **argv)
{
    const bool no_gpu = argc > 1 && !std::strcmp(argv[1], "--no-gpu");
    host_paths();
    if (!no_gpu)
        gpu_paths();
    std::printf("%s (%d failed checks)\n", failures ? "FAILED" : "PASSED", failures);
    return failures ? 1 : 0;
}
