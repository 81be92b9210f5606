// Bit-plane packing launchers with the reference's signatures (engine/common/pack.h:20-24).
// in_data / pack_data are device pointers; the return value is the HIP status of the launch.
#pragma once
#include "common/base.h"

inline hipError_t abq_shim_pack_status(abq_status s)
{
    if (s == ABQ_OK)
        return hipSuccess;
    const int e = abq_last_hip_error();
    return s == ABQ_ERR_LAUNCH && e ? (hipError_t)e : hipErrorInvalidValue;
}

// nibble-packed input, eight 4-bit elements per int (first element in the top nibble)
inline hipError_t launch_pack4(const int *in_data, int *pack_data, int m, int k, int BIT, hipStream_t stream = 0)
{
    return abq_shim_pack_status(abq_pack_u4(reinterpret_cast<const uint32_t *>(in_data),
                                            reinterpret_cast<uint32_t *>(pack_data), m, k, BIT, stream));
}

// one int32 per element
inline hipError_t launch_pack(const int *in_data, int *pack_data, int m, int k, int BIT, hipStream_t stream = 0)
{
    return abq_shim_pack_status(abq_pack_i32(in_data, reinterpret_cast<uint32_t *>(pack_data), m, k, BIT, stream));
}
