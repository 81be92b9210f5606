// First-generation entry point (reference: engine/wmma_any/wmma_any.h:18-38, wmma_any.cu:28-87):
// one call that sizes, configures and launches the GEMM, int32 output.
#pragma once
#include "common/base.h"

struct AnyQuantParams {
    const int *X;
    const int *W;
    const half *C;
    int *D;
    bool bias = false;
    const int M;
    const int N;
    const int K;
};

template <typename QuantType, typename ThreadBlockShape, typename WarpShape, typename MmaShape, int kThreadBlockStage>
hipError_t launchWmmaAnyKernel(const AnyQuantParams &params, const hipStream_t &stream)
{
    const abq_tile_config cfg =
        abq_shim::tile_config<QuantType, ThreadBlockShape, WarpShape, MmaShape, kThreadBlockStage>();
    const abq_status rc = abq_gemm_launch(&cfg, reinterpret_cast<const uint32_t *>(params.X),
                                          reinterpret_cast<const uint32_t *>(params.W), params.C, params.D,
                                          params.bias ? 1 : 0, params.M, params.N, params.K, stream);
    if (rc == ABQ_OK)
        return hipSuccess;
    const int e = abq_last_hip_error();
    return rc == ABQ_ERR_LAUNCH && e ? (hipError_t)e : hipErrorInvalidValue;
}
