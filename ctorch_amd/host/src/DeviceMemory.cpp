// HBM behind Storage: allocation through the C ABI, recycled by a size-bucketed pool.
// Every operator result in this front-end is a fresh tensor (as in the reference, where each
// kernel returns a new Tensor: src/kernels/CPU-BASIC/Add_BASIC_kernel.cpp:44); without a pool each
// op would pay a hipMalloc and - worse - a hipFree, which synchronises the device.  Buckets are
// 2^k * {1, 1.25, 1.5, 1.75}, at most 25 % over the request; freed blocks are kept until
// device_trim().  Launches outside a graph recording go to the null stream, and graph replays go to
// one blocking stream that the null stream orders itself with, so a block handed out again is only
// touched after every kernel that used it before; what a recording allocates stays reserved for
// its graph (BlockReservation) and is never handed to anyone else while the graph lives.
#include <cstdio>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "Storage.h"
#include "kernels.h"
#include "ctorch_amd.h"

namespace ctorch_amd_host {

struct BlockReservation {
    std::unordered_map<size_t, std::vector<void*>> parked;   // bucket -> released blocks of this graph
    std::vector<void*> blocks;                                // every block acquired while recording
};

namespace {

thread_local BlockReservation* t_reserving = nullptr;

struct Pool {
    std::mutex mu;
    std::unordered_map<size_t, std::vector<void*>> free_lists;
    size_t cached_bytes = 0;
    // blocks that a recorded graph refers to: released ones are parked with their graph instead of
    // going back to the free lists, so that nothing else is handed memory a replay will write
    std::unordered_map<void*, BlockReservation*> owner;
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

thread_local void* t_stream = nullptr;
thread_local bool t_recording = false;

void no_host_wait(const char* what) {
    if (t_recording)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::TENSOR_STATE,
                                     std::string(what) + ": the host cannot wait for the device while a graph is being recorded");
}

[[noreturn]] void die(const char* what, int rc) {
    Ctorch_Error::throwException(ErrorPlatform::kAMD, rc == CTAMD_ENOMEM ? ErrorType::MEMORY : ErrorType::PLATFORM_API,
                                 std::string(what) + ": " + ctamd_last_error());
}

}  // namespace

void* current_stream() { return t_stream; }
void set_current_stream(void* stream) { t_stream = stream; }
bool recording() { return t_recording; }
void set_recording(bool on) { t_recording = on; }

void init_device() {
    static std::once_flag once;
    static int rc = 0;
    std::call_once(once, [] { rc = ctamd_init(0); });
    if (rc != CTAMD_OK) die("ctamd_init", rc);
}

void* device_acquire(size_t bytes) {
    init_device();
    size_t b = bucket(bytes);
    BlockReservation* res = t_reserving;
    {
        std::lock_guard<std::mutex> lock(pool().mu);
        if (res) {                              // recording: first the blocks this graph already owns
            auto it = res->parked.find(b);
            if (it != res->parked.end() && !it->second.empty()) {
                void* p = it->second.back();
                it->second.pop_back();
                return p;
            }
        }
        auto it = pool().free_lists.find(b);
        if (it != pool().free_lists.end() && !it->second.empty()) {
            void* p = it->second.back();
            it->second.pop_back();
            pool().cached_bytes -= b;
            if (res) {
                pool().owner[p] = res;
                res->blocks.push_back(p);
            }
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
    if (res) {
        std::lock_guard<std::mutex> lock(pool().mu);
        pool().owner[p] = res;
        res->blocks.push_back(p);
    }
    return p;
}

BlockReservation* reservation_begin() {
    BlockReservation* r = new BlockReservation();
    t_reserving = r;
    return r;
}
void reservation_stop() { t_reserving = nullptr; }
void reservation_destroy(BlockReservation* r) {
    if (!r) return;
    if (t_reserving == r) t_reserving = nullptr;
    {
        std::lock_guard<std::mutex> lock(pool().mu);
        for (void* p : r->blocks) pool().owner.erase(p);        // live ones return to the free lists when released
        for (auto& kv : r->parked) {
            auto& fl = pool().free_lists[kv.first];
            fl.insert(fl.end(), kv.second.begin(), kv.second.end());
            pool().cached_bytes += kv.first * kv.second.size();
        }
    }
    delete r;
}

void device_release(void* p, size_t bytes) {
    if (!p) return;
    size_t b = bucket(bytes);
    std::lock_guard<std::mutex> lock(pool().mu);
    auto own = pool().owner.find(p);
    if (own != pool().owner.end()) {
        own->second->parked[b].push_back(p);
        return;
    }
    pool().free_lists[b].push_back(p);
    pool().cached_bytes += b;
}

void device_trim() {
    no_host_wait("device_trim");          // throws while a graph is being recorded: before anything is taken off the lists
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
    no_host_wait("host-to-device copy");
    int rc = ctamd_memcpy_h2d(dst, src, bytes, t_stream);
    if (rc == CTAMD_OK) rc = ctamd_sync(t_stream);   // the host buffer may be reused at once
    if (rc != CTAMD_OK) die("ctamd_memcpy_h2d", rc);
}
void device_copy_d2h(void* dst, const void* src, size_t bytes) {
    no_host_wait("device-to-host copy");
    if (bytes <= CTAMD_READ_SMALL_MAX) {       // a loss, a flag: one queued copy and one wait
        int rc = ctamd_read_small(dst, src, bytes, t_stream);
        if (rc != CTAMD_OK) die("ctamd_read_small", rc);
        return;
    }
    int rc = ctamd_memcpy_d2h(dst, src, bytes, t_stream);
    if (rc == CTAMD_OK) rc = ctamd_sync(t_stream);
    if (rc != CTAMD_OK) die("ctamd_memcpy_d2h", rc);
}
void device_copy_d2d(void* dst, const void* src, size_t bytes) {
    int rc = ctamd_memcpy_d2d(dst, src, bytes, t_stream);
    if (rc != CTAMD_OK) die("ctamd_memcpy_d2d", rc);
}
void device_sync() {
    no_host_wait("device_sync");
    int rc = ctamd_sync(t_stream);
    if (rc != CTAMD_OK) die("ctamd_sync", rc);
}

}  // namespace ctorch_amd_host
