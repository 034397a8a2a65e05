// The plainest BaseAllocator: every request goes straight to hipMalloc / hipHostMalloc and every
// release to hipFree / hipHostFree.  Enough to drive the layer code from tests and benchmarks; a
// serving process would pass its own pooling implementation of the same interface.
#pragma once
#include "src/memory/allocator/base_allocator.h"
#include "src/utils/macro.h"

class HipAllocator : public BaseAllocator {
public:
    void* UnifyMalloc(void* ptr, size_t size, bool is_host = false) override {
        (void)ptr;
        void* out = nullptr;
        if (size == 0) return nullptr;
        if (is_host) CHECK(hipHostMalloc(&out, size));
        else CHECK(hipMalloc(&out, size));
        return out;
    }
    void UnifyFree(void* ptr, bool is_host = false) override {
        if (ptr == nullptr) return;
        if (is_host) CHECK(hipHostFree(ptr));
        else CHECK(hipFree(ptr));
    }
};
