// Shared host-side vocabulary of the engine API: shapes, quantisation type, the naming macros
// that turn a tile tuple into the pair of function-pointer globals callers link against.
// Mirrors the public part of the reference's engine/common/base.h (:30-43 types, :138-166
// macros); the device-side helpers of that file (swizzles, cp.async pipeline, IntVector) have
// no counterpart here because the gfx950 kernels live behind the C ABI.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cassert>
#include <iostream>
#include <string>

#include "abq_gemm.h"

#define CEIL(x, y) (((x) + (y)-1) / (y))
#define ROUND_UP(x, y) ((CEIL((x), (y))) * (y))

typedef _Float16 half; // fp16 as the gfx950 compiler spells it

template <int M_, int N_, int K_> struct ShapeBase {
    static constexpr int M = M_, N = N_, K = K_;
};

template <int X_BITS_, int W_BITS_, bool SIGNED_> struct QuantType {
    static constexpr int X_BITS = X_BITS_, W_BITS = W_BITS_;
    static constexpr bool SIGNED = SIGNED_;
};

namespace abq_shim {

template <typename QuantType, typename CtaShape, typename WarpShape, typename MmaShape, int NStage>
inline abq_tile_config tile_config()
{
    return abq_tile_config{ QuantType::X_BITS, QuantType::W_BITS, QuantType::SIGNED ? 1 : 0,
                            CtaShape::M,       CtaShape::N,       CtaShape::K,
                            WarpShape::M,      WarpShape::N,      WarpShape::K,
                            MmaShape::M,       MmaShape::N,       MmaShape::K,
                            NStage };
}

// Shared by both name families: fills the caller-visible state from the library's answer.

template <typename State>
inline State make_state(const abq_tile_config &cfg, int *X, int *W, int M, int N, int K, void *D, half *C,
                        bool bias, int out_kind)
{
    // the reference asserts; a release build of it would go on and ignore the flag
    assert(!bias && "Bias operation is not supported temporarily\n");
    State st;
    st.args = typename State::Argument_t{ M, N, K, X, W, C, reinterpret_cast<decltype(st.args.D)>(D), bias };
    const abq_status rc = abq_gemm_init(&cfg, 0, 0, 0, reinterpret_cast<const uint32_t *>(X),
                                        reinterpret_cast<const uint32_t *>(W), M, N, K, D, C, bias ? 1 : 0,
                                        out_kind, &st.native);
    if (rc != ABQ_OK) {
        std::cerr << "Init failed: " << abq_status_string(rc) << std::endl;
        st.initSuccess = false;
        return st;
    }
    st.shared_mem_size = st.native.shared_mem_size;
    st.gridDim = dim3(st.native.grid_dim.x, st.native.grid_dim.y, st.native.grid_dim.z);
    st.blockDim = dim3(st.native.block_dim.x, st.native.block_dim.y, st.native.block_dim.z);
    st.initSuccess = true;
    return st;
}

} // namespace abq_shim

// ---- naming: type_XxWxSIGNED_BMxBNxBK_WMxWNxWK_MMxMNxMK_NSTAGE_{Init,Exec}Fn -------------------
#define AQ_INIT_FUN(type) type##InitFn_t
#define AQ_EXEC_FUN(type) type##ExecFn_t
#define AQ_OP_STATE(type) type##OpState

#define AQ_NAME_FUN(type, fn, X_BITS, W_BITS, SIGNED, BLOCK_M, BLOCK_N, BLOCK_K, WARP_M, WARP_N, WARP_K, MMA_M, \
                    MMA_N, MMA_K, NSTAGE)                                                                       \
    type##_##X_BITS##x##W_BITS##x##SIGNED##_##BLOCK_M##x##BLOCK_N##x##BLOCK_K##_##WARP_M##x##WARP_N##x##WARP_K##_##MMA_M##x##MMA_N##x##MMA_K##_##NSTAGE##_##fn##Fn

#define AQ_TEMPLATE_ARGS_(X_BITS, W_BITS, SIGNED, BLOCK_M, BLOCK_N, BLOCK_K, WARP_M, WARP_N, WARP_K, MMA_M, MMA_N, \
                          MMA_K, NSTAGE)                                                                           \
    QuantType<X_BITS, W_BITS, SIGNED>, ShapeBase<BLOCK_M, BLOCK_N, BLOCK_K>, ShapeBase<WARP_M, WARP_N, WARP_K>,     \
        ShapeBase<MMA_M, MMA_N, MMA_K>, NSTAGE

// Defines the two globals of one configuration.
#define AQ_INSTANTIATE_FUN(type, ...)                                                    \
    type##InitFn_t AQ_NAME_FUN(type, Init, __VA_ARGS__) = type##InitFn<AQ_TEMPLATE_ARGS_(__VA_ARGS__)>; \
    type##ExecFn_t AQ_NAME_FUN(type, Exec, __VA_ARGS__) = type##ExecFn<AQ_TEMPLATE_ARGS_(__VA_ARGS__)>;

// Declares them.
#define AQ_DECL_FUN(type, ...)                                   \
    extern type##InitFn_t AQ_NAME_FUN(type, Init, __VA_ARGS__);  \
    extern type##ExecFn_t AQ_NAME_FUN(type, Exec, __VA_ARGS__);
