// Host launch state and the Init / Exec function families of the engine API
// (reference: engine/mma_any/aq_wmma_op.h:19-32 state, :147-170 functions and typedefs).
//
// InitFn captures the arguments and resolves the tile tuple named by its template parameters to
// a gfx950 kernel through the C ABI (abq_gemm_init); ExecFn launches it (abq_gemm_exec).  The
// reference's tensor-core tuples (MMA 8x8x128, 16x8x128, 16x8x256) resolve to the library's own
// choice for the shape; native tuples select exactly the named kernel.
#pragma once
#include "common/base.h"

struct AqBWMMAOpState {
    size_t shared_mem_size = 0;
    dim3 gridDim;
    dim3 blockDim;
    bool initSuccess = false;
    struct Argument_t {
        int M, N, K;
        int *X;
        int *W;
        half *C;
        int *D;
        bool bias = false;
    } args;
    abq_gemm_state native; // what ExecFn hands to the library
};

template <typename QuantType, typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage>
AqBWMMAOpState AqBWMMAInitFn(int *X, int *W, int M, int N, int K, int *D, half *C, bool bias)
{
    return abq_shim::make_state<AqBWMMAOpState>(
        abq_shim::tile_config<QuantType, ThreadBlockShape, WarpShape, MmaShape, NStage>(), X, W, M, N, K, D, C, bias,
        ABQ_OUT_I32);
}

template <typename QuantType, typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage>
void AqBWMMAExecFn(AqBWMMAOpState &state, hipStream_t stream = NULL)
{
    // like the reference, errors surface through hipGetLastError() / the next synchronisation
    (void)abq_gemm_exec(&state.native, stream);
}

typedef AqBWMMAOpState (*AqBWMMAInitFn_t)(int *, int *, int, int, int, int *, half *, bool);
typedef void (*AqBWMMAExecFn_t)(AqBWMMAOpState &, hipStream_t);
