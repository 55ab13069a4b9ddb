// Small RAII helpers over the C ABI for the C++ host classes: status -> exception, device and pinned
// buffers that grow on demand, a stream, and host/device pointer staging.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>

#include "ahpc_hip.h"
#include "api/attention_interface.hpp"

namespace attention_hpc {
namespace hipsup {

inline int dtype_code(DataType t) { return static_cast<int>(t); }  // enumerators match AHPC_F32/F16/BF16
inline size_t dtype_size(DataType t) { return t == DataType::FLOAT32 ? 4 : 2; }

// Non-zero C-ABI status -> AttentionException.  Rejected arguments map to INVALID_INPUT /
// UNSUPPORTED_OPERATION, device errors to COMPUTATION_FAILED (the reference's CUDA_CHECK,
// src/backends/cuda/cuda_flash_attention.hpp:16-22), allocation failures to MEMORY_ALLOCATION_FAILED.
inline void check(int status, const char* what, bool is_alloc = false) {
    if (status == 0) return;
    AttentionError code = AttentionError::COMPUTATION_FAILED;
    if (status == AHPC_ERR_UNSUPPORTED_HEAD_DIM || status == AHPC_ERR_UNSUPPORTED_GROUP) code = AttentionError::UNSUPPORTED_OPERATION;
    else if (status == AHPC_ERR_NO_DEVICE) code = AttentionError::BACKEND_NOT_AVAILABLE;
    else if (status < 0) code = AttentionError::INVALID_INPUT;
    else if (is_alloc) code = AttentionError::MEMORY_ALLOCATION_FAILED;
    throw AttentionException(code, std::string("HIP: ") + what + ": " + ahpc_hip_error_string(status));
}

class DeviceBuffer {
public:
    DeviceBuffer() = default;
    ~DeviceBuffer() { release(); }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    // Ensures at least `bytes`; contents are NOT preserved when it has to grow.
    void* reserve(size_t bytes) {
        if (bytes > size_) {
            release();
            check(ahpc_hip_malloc(&ptr_, bytes), "device allocation", true);
            size_ = bytes;
        }
        return ptr_;
    }
    void release() {
        if (ptr_) ahpc_hip_free(ptr_);
        ptr_ = nullptr;
        size_ = 0;
    }
    void* get() const { return ptr_; }
    size_t size() const { return size_; }

private:
    void* ptr_ = nullptr;
    size_t size_ = 0;
};

class PinnedBuffer {
public:
    PinnedBuffer() = default;
    ~PinnedBuffer() { release(); }
    PinnedBuffer(const PinnedBuffer&) = delete;
    PinnedBuffer& operator=(const PinnedBuffer&) = delete;
    void* reserve(size_t bytes) {
        if (bytes > size_) {
            release();
            check(ahpc_hip_host_malloc(&ptr_, bytes), "pinned host allocation", true);
            size_ = bytes;
        }
        return ptr_;
    }
    void release() {
        if (ptr_) ahpc_hip_host_free(ptr_);
        ptr_ = nullptr;
        size_ = 0;
    }
    void* get() const { return ptr_; }

private:
    void* ptr_ = nullptr;
    size_t size_ = 0;
};

// Created at first use, so that objects can be constructed (and queried) on a machine without a GPU.
class Stream {
public:
    Stream() = default;
    ~Stream() {
        if (s_) ahpc_hip_stream_destroy(s_);
    }
    Stream(const Stream&) = delete;
    Stream& operator=(const Stream&) = delete;
    void* get() {
        if (!s_) check(ahpc_hip_stream_create(&s_), "stream create");
        return s_;
    }
    void sync() { check(ahpc_hip_stream_synchronize(get()), "stream synchronize"); }

private:
    void* s_ = nullptr;
};

inline bool is_device_pointer(const void* p) {
    int dev = 0;
    check(ahpc_hip_ptr_is_device(p, &dev), "pointer query");
    return dev != 0;
}

// Milliseconds between two points of a stream, measured with events.
class EventTimer {
public:
    EventTimer() {
        check(ahpc_hip_event_create(&a_), "event create");
        check(ahpc_hip_event_create(&b_), "event create");
    }
    ~EventTimer() {
        ahpc_hip_event_destroy(a_);
        ahpc_hip_event_destroy(b_);
    }
    void start(void* stream) { check(ahpc_hip_event_record(a_, stream), "event record"); }
    void stop(void* stream) { check(ahpc_hip_event_record(b_, stream), "event record"); }
    double elapsed_ms() {
        float ms = 0.0f;
        check(ahpc_hip_event_synchronize(b_), "event synchronize");
        check(ahpc_hip_event_elapsed_ms(a_, b_, &ms), "event elapsed");
        return ms;
    }

private:
    void* a_ = nullptr;
    void* b_ = nullptr;
};

}  // namespace hipsup
}  // namespace attention_hpc
