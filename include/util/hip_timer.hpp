// hipEvent stopwatch; same contract as the reference's util/cuda_timer.hpp:13-42
// (start() then stop() returns elapsed milliseconds), but stream-aware.
#pragma once

#include "hip_utils.hpp"

namespace tiledcuda {

class HipTimer {
  public:
    HipTimer() {
        HipCheck(hipEventCreate(&start_));
        HipCheck(hipEventCreate(&stop_));
    }
    ~HipTimer() {
        (void)hipEventDestroy(start_);
        (void)hipEventDestroy(stop_);
    }
    HipTimer(const HipTimer&) = delete;
    HipTimer& operator=(const HipTimer&) = delete;

    void start(hipStream_t stream = nullptr) {
        stream_ = stream;
        HipCheck(hipEventRecord(start_, stream_));
    }

    float stop() {
        HipCheck(hipEventRecord(stop_, stream_));
        HipCheck(hipEventSynchronize(stop_));
        float ms = 0.f;
        HipCheck(hipEventElapsedTime(&ms, start_, stop_));
        return ms;
    }

  private:
    hipEvent_t start_{}, stop_{};
    hipStream_t stream_{nullptr};
};

}  // namespace tiledcuda
