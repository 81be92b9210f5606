// Defines the globals aq_wmma_library.h declares (reference: engine/mma_any/aq_wmma_library.cu
// and aq_bmma_impl/aq_bmma_w*.cu).  Host code only: each global is a pointer to a host template
// that forwards its tile tuple to the C ABI.
#include "mma_any/aq_wmma_op.h"

#define AQ_CONFIG(...) AQ_INSTANTIATE_FUN(AqBWMMA, __VA_ARGS__)
#include "mma_any/aq_wmma_library.h"
#undef AQ_CONFIG

// The two production tiles of the FT wrapper, by their reference names
// (abq_gemm_wrapper.cu:106-124); they resolve to the library's choice for the shape.
AQ_INSTANTIATE_FUN(AqBWMMA, 8, 2, true, 1, 48, 512, 8, 24, 128, 8, 8, 128, 4)
AQ_INSTANTIATE_FUN(AqBWMMA, 8, 2, false, 1, 48, 512, 8, 24, 128, 8, 8, 128, 4)
AQ_INSTANTIATE_FUN(AqBWMMA, 8, 2, true, 8, 48, 256, 32, 48, 128, 8, 8, 128, 5)
AQ_INSTANTIATE_FUN(AqBWMMA, 8, 2, false, 8, 48, 256, 32, 48, 128, 8, 8, 128, 5)
