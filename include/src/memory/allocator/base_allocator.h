// The allocator interface the reference's model and layers are handed
// (src/memory/allocator/base_allocator.h:5-19): same names and signatures, HIP underneath.  Only the
// interface is part of this library's boundary -- the context-decoder layer takes its activation
// buffers from whatever implementation the caller passes; the reference's pooling allocator
// (cuda_allocator.h) is not rebuilt.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>

class BaseAllocator {
public:
    virtual ~BaseAllocator() {}

    template <typename T>
    T* Malloc(T* ptr, size_t size, bool is_host) {
        return static_cast<T*>(UnifyMalloc(static_cast<void*>(ptr), size, is_host));
    }
    virtual void* UnifyMalloc(void* ptr, size_t size, bool is_host = false) = 0;

    template <typename T>
    void Free(T* ptr, bool is_host = false) {
        UnifyFree(static_cast<void*>(ptr), is_host);
    }
    virtual void UnifyFree(void* ptr, bool is_host = false) = 0;
};
