// Event timer of the benchmark programs (reference: block_sparse/benchmark/timing_util.h:3-36),
// on the null stream like the reference's.
#pragma once
#include <hip/hip_runtime.h>

struct GpuTimer {
    hipEvent_t startEvent, stopEvent;
    GpuTimer()
    {
        (void)hipEventCreate(&startEvent);
        (void)hipEventCreate(&stopEvent);
    }
    ~GpuTimer()
    {
        (void)hipEventDestroy(startEvent);
        (void)hipEventDestroy(stopEvent);
    }
    void start() { (void)hipEventRecord(startEvent, 0); }
    void stop()
    {
        (void)hipEventRecord(stopEvent, 0);
        (void)hipEventSynchronize(stopEvent);
    }
    float elapsed_msecs()
    {
        float elapsed = 0.f;
        (void)hipEventElapsedTime(&elapsed, startEvent, stopEvent);
        return elapsed;
    }
};
