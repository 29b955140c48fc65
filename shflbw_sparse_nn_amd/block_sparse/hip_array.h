// Host vector + device buffer pair used by tests, examples and benchmarks; the gfx950
// counterpart of block_sparse/cuda_array.h:5-87 (same members and method names).
#pragma once
#include <cstdlib>
#include <vector>
#include "hip_error.h"

template <typename T>
struct HipArray {
    int size = 0;
    std::vector<T> host_array;
    T* device_ptr = nullptr;
    bool initialized = false;
    bool device_synced = false;

    virtual void __fill() {}
    virtual ~HipArray() { release(); }

    // allocate `size_` elements on host and device, fill the host side, upload
    void initialize(int size_)
    {
        release();
        size = size_;
        host_array.assign(size_, T());
        if (size_ > 0) {
            __fill();
            HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&device_ptr), sizeof(T) * size_));
            sync_device();
        }
        initialized = true;
    }
    // host-only copy of an existing vector
    void initialize(const std::vector<T>& that)
    {
        host_array = that;
        size = static_cast<int>(that.size());
        initialized = true;
    }
    void sync_device()
    {
        if (size == 0) return;
        HIP_CHECK(hipMemcpy(device_ptr, host_array.data(), sizeof(T) * size, hipMemcpyHostToDevice));
        device_synced = true;
    }
    void sync_host()
    {
        if (size == 0) return;
        HIP_CHECK(hipMemcpy(host_array.data(), device_ptr, sizeof(T) * size, hipMemcpyDeviceToHost));
    }
    std::vector<T>& host_ref() { return host_array; }
    T* device_data() { return device_ptr; }

private:
    void release()
    {
        if (device_ptr) {
            HIP_CHECK(hipFree(device_ptr));
            device_ptr = nullptr;
        }
    }
};

// small integers in [-4, 4] from the C library generator (cuda_array.h:62-69)
template <typename T>
struct HipRandomArray : public HipArray<T> {
    void __fill() override
    {
        for (auto& x : this->host_array) x = static_cast<T>(static_cast<float>(std::rand() % 9 - 4));
    }
};
template <typename T>
struct HipZerosArray : public HipArray<T> {
    void __fill() override
    {
        for (auto& x : this->host_array) x = static_cast<T>(0.0f);
    }
};
template <typename T>
struct HipOnesArray : public HipArray<T> {
    void __fill() override
    {
        for (auto& x : this->host_array) x = static_cast<T>(1.0f);
    }
};
