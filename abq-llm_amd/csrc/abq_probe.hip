// Measurement aids: what a launch and a plain read of a buffer cost on this device, the floor a decode GEMM
// (one launch over a few MB of weights) is compared with; and what the matrix cores sustain in a loop that
// touches nothing but registers, on operand bits the caller chooses (the clock of the matrix cores follows the
// power their data makes them draw: the rate on random bits is the ceiling of a GEMM on such data, not the
// datasheet figure).  No counterpart in the reference.
#include "abq_probe.h"

#include <hip/hip_runtime.h>

namespace abq {

__global__ void probe_empty_kernel(int *out)
{
    if (out == reinterpret_cast<int *>(1))
        *out = 0;
}

// every lane reads one 16-byte piece, coalesced; nothing is computed and nothing written (the store below
// never happens for data that is not all ones)
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4 *__restrict__ p, size_t n16, int *out)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) {
        const uint4 v = p[i];
        if ((v.x & v.y & v.z & v.w) == 0xFFFFFFFFu && out)
            out[0] = 1;
    }
}

typedef int v4i_p __attribute__((ext_vector_type(4)));
typedef int v8i_p __attribute__((ext_vector_type(8)));
typedef int v16i_p __attribute__((ext_vector_type(16)));
typedef float v16f_p __attribute__((ext_vector_type(16)));

// Eight waves per compute unit (two per SIMD), four independent accumulator tiles per wave, two operand sets
// used in turn; operands come from `data` (8 KiB: 2 sets x (A, B) x 64 lanes x 32 bytes) and never change.
template <bool FP6>
__global__ __launch_bounds__(256) void probe_mfma_kernel(const uint32_t *__restrict__ data, int n, float *out)
{
    const int lane = threadIdx.x & 63;
    v8i_p ops[4]; // set 0: A, B; set 1: A, B
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int d = 0; d < 8; ++d)
            ops[i][d] = (int)data[(i * 64 + lane) * 8 + d];
    if constexpr (FP6) {
        v16f_p acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[t][e] = 0.f;
        for (int it = 0; it < n; it += 8)
#pragma unroll
            for (int u = 0; u < 8; ++u)
                acc[u & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ops[2 * (u >> 2)], ops[2 * (u >> 2) + 1], acc[u & 3], 2, 2, 0, 0, 0, 0);
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            sum += acc[t][0] + acc[t][15];
        if (out)
            out[blockIdx.x * 256 + threadIdx.x] = sum;
    } else {
        v16i_p acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[t][e] = 0;
        for (int it = 0; it < n; it += 8)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const v8i_p &a = ops[2 * (u >> 2)], &b = ops[2 * (u >> 2) + 1];
                acc[u & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(v4i_p{ a[0], a[1], a[2], a[3] }, v4i_p{ b[0], b[1], b[2], b[3] }, acc[u & 3], 0, 0, 0);
            }
        int sum = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            sum += acc[t][0] + acc[t][15];
        if (out)
            out[blockIdx.x * 256 + threadIdx.x] = (float)sum;
    }
}

} // namespace abq

extern "C" abq_status abq_probe_launch(int kind, const void *buf, size_t bytes, void *stream)
{
    if (kind == ABQ_PROBE_EMPTY) {
        hipLaunchKernelGGL(abq::probe_empty_kernel, dim3(256), dim3(256), 0, (hipStream_t)stream, nullptr);
    } else if (kind == ABQ_PROBE_READ) {
        if (!buf || bytes < 16)
            return ABQ_ERR_INVALID_ARG;
        const size_t n16 = bytes / 16;
        const size_t blocks = (n16 + 255) / 256;
        if (blocks >= (1ull << 31))
            return ABQ_ERR_TOO_LARGE;
        hipLaunchKernelGGL(abq::probe_read_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           static_cast<const uint4 *>(buf), n16, nullptr);
    } else if (kind == ABQ_PROBE_MFMA_I8 || kind == ABQ_PROBE_MFMA_FP6) {
        // bytes: matrix-core instructions per wave
        if (!buf || bytes < 8 || bytes % 8 != 0 || bytes > (1u << 30))
            return ABQ_ERR_INVALID_ARG;
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            return ABQ_ERR_LAUNCH;
        if (kind == ABQ_PROBE_MFMA_I8)
            hipLaunchKernelGGL(abq::probe_mfma_kernel<false>, dim3(2 * cus), dim3(256), 0, (hipStream_t)stream,
                               static_cast<const uint32_t *>(buf), (int)bytes, nullptr);
        else
            hipLaunchKernelGGL(abq::probe_mfma_kernel<true>, dim3(2 * cus), dim3(256), 0, (hipStream_t)stream,
                               static_cast<const uint32_t *>(buf), (int)bytes, nullptr);
    } else {
        return ABQ_ERR_INVALID_ARG;
    }
    return hipGetLastError() == hipSuccess ? ABQ_OK : ABQ_ERR_LAUNCH;
}
