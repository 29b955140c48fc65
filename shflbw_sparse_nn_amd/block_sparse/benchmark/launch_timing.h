// Timing of an operator for the benchmark programs: the mean duration of `repeat` launches issued back to
// back on one stream after `warmup` untimed ones, measured with two events on that same stream (the
// reference's method: 10 warm-ups and 100 launches, block_sparse/benchmark/benchmark.spmm.cu:29-50).
#pragma once
#include <hip/hip_runtime.h>
#include <iostream>

namespace launch_timing {

// two events recorded on the stream the launches go to; valid() is false when they could not be created
class StreamInterval {
public:
    explicit StreamInterval(hipStream_t s) : stream_(s)
    {
        ok_ = hipEventCreate(&first_) == hipSuccess;
        ok_ = ok_ && hipEventCreate(&last_) == hipSuccess;
    }
    StreamInterval(const StreamInterval&) = delete;
    StreamInterval& operator=(const StreamInterval&) = delete;
    ~StreamInterval()
    {
        if (first_) (void)hipEventDestroy(first_);
        if (last_) (void)hipEventDestroy(last_);
    }
    bool valid() const { return ok_; }
    bool open() { return ok_ && hipEventRecord(first_, stream_) == hipSuccess; }
    // milliseconds between open() and now, after everything in between has finished; negative on failure
    float close()
    {
        float ms = -1.f;
        if (!ok_ || hipEventRecord(last_, stream_) != hipSuccess || hipEventSynchronize(last_) != hipSuccess ||
            hipEventElapsedTime(&ms, first_, last_) != hipSuccess)
            return -1.f;
        return ms;
    }

private:
    hipStream_t stream_;
    hipEvent_t first_ = nullptr, last_ = nullptr;
    bool ok_ = false;
};

// true when the device is idle and no launch so far has left an error behind; says so otherwise
inline bool device_clean(const char* when)
{
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) return true;
    std::cerr << "device error " << when << ": " << hipGetErrorString(e) << std::endl;
    return false;
}

// Mean milliseconds per launch, or -1: one launch checked on its own first (a kernel that faults should not
// be timed a hundred times), then warmup + repeat launches with the interval around the last `repeat`.
template <typename Launch>
float mean_launch_ms(Launch&& launch, hipStream_t stream, int warmup, int repeat)
{
    launch();
    if (!device_clean("after the first launch")) return -1.f;
    StreamInterval interval(stream);
    for (int i = 0; i < warmup; i++) launch();
    if (!interval.open()) return -1.f;
    for (int i = 0; i < repeat; i++) launch();
    const float total = interval.close();
    if (total < 0.f || !device_clean("after the timed launches")) return -1.f;
    return total / repeat;
}

} // namespace launch_timing
