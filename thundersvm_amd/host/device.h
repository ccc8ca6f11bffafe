// Device memory and error plumbing of the host layer.  DeviceBuffer<T> is the native replacement
// for the reference's SyncArray<T> on this path: it owns device memory only, and every transfer is
// an explicit call (the reference's implicit host_data()/device_data() mirroring,
// src/thundersvm/syncmem.cpp:58-108, is what forces a device-host round trip per solver iteration).
#pragma once
#include <mutex>
#include <hip/hip_runtime.h>

#include <new>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/thundersvm_amd.h"

namespace tsvm {

inline void hip_check(hipError_t e, const char *what) {
    if (e == hipSuccess) return;
    if (e == hipErrorOutOfMemory) throw std::bad_alloc();   // include/thundersvm/util/common.h:33-39
    throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
#define TSVM_HIP_CHECK(expr) ::tsvm::hip_check((expr), #expr)

// Status of a C-ABI kernel call -> exception (2 == hipErrorOutOfMemory).
inline void abi_check(int rc) {
    if (rc == 0) return;
    if (rc == 2) throw std::bad_alloc();
    throw std::runtime_error(std::string("thundersvm_amd kernel call failed: ") + tsvm_last_error());
}

size_t &device_bytes_in_use();   // running total of DeviceBuffer allocations (the SyncMem byte counter's role)

// One grow-only device allocation that outlives individual solves and holds the kernel rows (working-set
// rows plus the row cache).  Releasing a multi-gigabyte allocation costs up to seconds on this platform,
// so the 21 one-vs-one solves of a 7-class problem must not each allocate and free their own pool.
// Not counted in device_bytes_in_use().
// One training or prediction call at a time per process: the row arena, the pooled CU-masked streams and the staging
// buffers are shared by all of them (the reference is not re-entrant either: one cuSPARSE handle, one SyncMem
// counter).  The model-level entry points hold this lock for their duration, so calls from several host threads
// take turns instead of sharing those buffers.
std::recursive_mutex &device_work_mutex();

class RowArena {
public:
    static RowArena &instance();
    // bytes a solve may use when the caller gave no explicit budget: nine tenths of what is free or already held
    size_t auto_budget();
    void *acquire(size_t bytes, bool auto_sized);
    void release();
    size_t capacity() const { return cap_; }

private:
    void *ptr_ = nullptr;
    size_t cap_ = 0;
    bool full_budget_ = false;
};

template <typename T>
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t count) { resize(count); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), count_(o.count_) { o.ptr_ = nullptr; o.count_ = 0; }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
        if (this != &o) { release(); ptr_ = o.ptr_; count_ = o.count_; o.ptr_ = nullptr; o.count_ = 0; }
        return *this;
    }
    ~DeviceBuffer() { release(); }

    void resize(size_t count) {
        if (count == count_) return;
        release();
        if (count) {
            TSVM_HIP_CHECK(hipMalloc((void **) &ptr_, count * sizeof(T)));
            device_bytes_in_use() += count * sizeof(T);
        }
        count_ = count;
    }
    void release() {
        if (ptr_) {
            (void) hipFree(ptr_);
            device_bytes_in_use() -= count_ * sizeof(T);
        }
        ptr_ = nullptr;
        count_ = 0;
    }
    T *data() { return ptr_; }
    const T *data() const { return ptr_; }
    size_t size() const { return count_; }
    // Gives the memory up without freeing it: for a device that has stopped answering, where hipFree would not return.
    void abandon() { ptr_ = nullptr; count_ = 0; }

    void upload(const T *host, size_t count, size_t offset = 0) {
        if (count) TSVM_HIP_CHECK(hipMemcpy(ptr_ + offset, host, count * sizeof(T), hipMemcpyHostToDevice));
    }
    void upload(const std::vector<T> &v) { resize(v.size()); upload(v.data(), v.size()); }
    void download(T *host, size_t count, size_t offset = 0) const {
        if (count) TSVM_HIP_CHECK(hipMemcpy(host, ptr_ + offset, count * sizeof(T), hipMemcpyDeviceToHost));
    }
    std::vector<T> to_host() const { std::vector<T> v(count_); download(v.data(), count_); return v; }
    void zero() { if (count_) TSVM_HIP_CHECK(hipMemset(ptr_, 0, count_ * sizeof(T))); }

private:
    T *ptr_ = nullptr;
    size_t count_ = 0;
};

// Page-locked host staging memory that only grows (hipHostMalloc; copies from it are asynchronous and run at
// the link's rate).
template <typename T>
class PinnedBuffer {
public:
    PinnedBuffer() = default;
    PinnedBuffer(const PinnedBuffer &) = delete;
    PinnedBuffer &operator=(const PinnedBuffer &) = delete;
    ~PinnedBuffer() { if (ptr_) (void) hipHostFree(ptr_); }
    void reserve(size_t count) {
        if (count <= count_) return;
        if (ptr_) (void) hipHostFree(ptr_);
        ptr_ = nullptr;
        count_ = 0;
        TSVM_HIP_CHECK(hipHostMalloc((void **) &ptr_, count * sizeof(T)));
        count_ = count;
    }
    T *data() { return ptr_; }
    size_t size() const { return count_; }

private:
    T *ptr_ = nullptr;
    size_t count_ = 0;
};

}  // namespace tsvm
