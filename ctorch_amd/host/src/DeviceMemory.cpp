// HBM behind Storage: allocation through the C ABI, recycled by a size-bucketed pool.
// Every operator result in this front-end is a fresh tensor (as in the reference, where each
// kernel returns a new Tensor: src/kernels/CPU-BASIC/Add_BASIC_kernel.cpp:44); without a pool each
// op would pay a hipMalloc and - worse - a hipFree, which synchronises the device.  Buckets are
// 2^k * {1, 1.25, 1.5, 1.75}, at most 25 % over the request; freed blocks are kept until
// device_trim().  All work is issued on the default stream, so a block handed out again is only
// touched after every kernel that used it before.
#include <cstdio>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "Storage.h"
#include "kernels.h"
#include "ctorch_amd.h"

namespace ctorch_amd_host {
namespace {

struct Pool {
    std::mutex mu;
    std::unordered_map<size_t, std::vector<void*>> free_lists;
    size_t cached_bytes = 0;
};
Pool& pool() {
    static Pool* p = new Pool();   // never destroyed: storages may be released during exit
    return *p;
}

size_t bucket(size_t bytes) {
    if (bytes <= 256) return 256;
    size_t p2 = 256;
    while (p2 * 2 <= bytes) p2 *= 2;          // p2 <= bytes < 2*p2
    for (int q = 0; q < 4; ++q) {
        size_t c = p2 + (p2 / 4) * q;
        if (c >= bytes) return c;
    }
    return p2 * 2;
}

[[noreturn]] void die(const char* what, int rc) {
    Ctorch_Error::throwException(ErrorPlatform::kAMD, rc == CTAMD_ENOMEM ? ErrorType::MEMORY : ErrorType::PLATFORM_API,
                                 std::string(what) + ": " + ctamd_last_error());
}

}  // namespace

void init_device() {
    static std::once_flag once;
    static int rc = 0;
    std::call_once(once, [] { rc = ctamd_init(0); });
    if (rc != CTAMD_OK) die("ctamd_init", rc);
}

void* device_acquire(size_t bytes) {
    init_device();
    size_t b = bucket(bytes);
    {
        std::lock_guard<std::mutex> lock(pool().mu);
        auto it = pool().free_lists.find(b);
        if (it != pool().free_lists.end() && !it->second.empty()) {
            void* p = it->second.back();
            it->second.pop_back();
            pool().cached_bytes -= b;
            return p;
        }
    }
    void* p = nullptr;
    int rc = ctamd_malloc(&p, b);
    if (rc == CTAMD_ENOMEM || (rc != CTAMD_OK && pool().cached_bytes)) {
        device_trim();                         // give cached blocks back and retry once
        rc = ctamd_malloc(&p, b);
    }
    if (rc != CTAMD_OK) die("ctamd_malloc", rc);
    return p;
}

void device_release(void* p, size_t bytes) {
    if (!p) return;
    size_t b = bucket(bytes);
    std::lock_guard<std::mutex> lock(pool().mu);
    pool().free_lists[b].push_back(p);
    pool().cached_bytes += b;
}

void device_trim() {
    std::vector<void*> all;
    {
        std::lock_guard<std::mutex> lock(pool().mu);
        for (auto& kv : pool().free_lists) {
            all.insert(all.end(), kv.second.begin(), kv.second.end());
            kv.second.clear();
        }
        pool().cached_bytes = 0;
    }
    if (all.empty()) return;
    ctamd_sync(nullptr);
    for (void* p : all) ctamd_free(p);
}

void device_copy_h2d(void* dst, const void* src, size_t bytes) {
    int rc = ctamd_memcpy_h2d(dst, src, bytes, nullptr);
    if (rc == CTAMD_OK) rc = ctamd_sync(nullptr);   // the host buffer may be reused at once
    if (rc != CTAMD_OK) die("ctamd_memcpy_h2d", rc);
}
void device_copy_d2h(void* dst, const void* src, size_t bytes) {
    int rc = ctamd_memcpy_d2h(dst, src, bytes, nullptr);
    if (rc == CTAMD_OK) rc = ctamd_sync(nullptr);
    if (rc != CTAMD_OK) die("ctamd_memcpy_d2h", rc);
}
void device_copy_d2d(void* dst, const void* src, size_t bytes) {
    int rc = ctamd_memcpy_d2d(dst, src, bytes, nullptr);
    if (rc != CTAMD_OK) die("ctamd_memcpy_d2d", rc);
}
void device_sync() {
    int rc = ctamd_sync(nullptr);
    if (rc != CTAMD_OK) die("ctamd_sync", rc);
}

}  // namespace ctorch_amd_host
