// Event timer with the interface of the reference's CudaTimer (engine/common/timer.h:19-53).
#pragma once
#include <hip/hip_runtime_api.h>

class HipTimer {
public:
    explicit HipTimer(hipStream_t stream = 0) : stream_(stream)
    {
        (void)hipEventCreate(&start_);
        (void)hipEventCreate(&stop_);
    }
    ~HipTimer()
    {
        (void)hipEventDestroy(start_);
        (void)hipEventDestroy(stop_);
    }
    void start() { (void)hipEventRecord(start_, stream_); }
    void stop() { (void)hipEventRecord(stop_, stream_); }
    float elapsed_msecs()
    {
        float ms = 0.f;
        (void)hipEventSynchronize(stop_);
        (void)hipEventElapsedTime(&ms, start_, stop_);
        return ms;
    }

private:
    hipStream_t stream_;
    hipEvent_t start_, stop_;
};
typedef HipTimer CudaTimer; // the name the reference's harness sources use
