// Device allocator of the KV pool backed by the kernel library's own runtime entry points
// (warp34_malloc / warp34_free, warp34_cuda.h:142-164 in the reference).  Kept apart from
// kv_host.cpp so that the host logic links and tests without a GPU runtime.
#include "kv_host.h"

namespace warp34_host {

namespace {
struct RuntimeAllocator final : DeviceAllocator {
    int alloc(int device_id, size_t bytes, uint64_t* addr) override {
        int rc = warp34_set_device(device_id);
        if (rc) return rc;
        void* p = nullptr;
        rc = warp34_malloc(&p, bytes);
        *addr = (uint64_t)(uintptr_t)p;
        return rc;
    }
    void release(int device_id, uint64_t addr) override {
        if (warp34_set_device(device_id) == 0) warp34_free((void*)(uintptr_t)addr);
    }
};
}  // namespace

DeviceAllocator& runtime_allocator() {
    static RuntimeAllocator a;
    return a;
}

}  // namespace warp34_host
