// Runtime side of the C ABI: device selection, HBM allocation, explicit transfers, error text.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "common.h"

namespace ctamd {

namespace {
thread_local char g_err[512] = "";
constexpr int kMaxDevices = 16;
std::mutex g_mu;
float* g_scratch[kMaxDevices] = {};
int g_cus[kMaxDevices] = {};

// Work counters (per process): what the operators launched since the last reset had to move and
// compute, and the time that work takes at the published peaks.
// (lock-free: every launcher adds to them on its way to the launch)
std::atomic<double> g_bytes{0.0}, g_flops{0.0}, g_ideal_s{0.0};
std::atomic<uint64_t> g_launches{0};
inline void add_to(std::atomic<double>& a, double v) {
    double seen = a.load(std::memory_order_relaxed);
    while (!a.compare_exchange_weak(seen, seen + v, std::memory_order_relaxed)) {}
}
std::atomic<int> g_math_mode{CTAMD_MATH_FAST};
constexpr double kHbmBytesPerS = 8.0e12;        // MI355X HBM3E
constexpr double kMfmaF32FlopPerS = 157.3e12;   // MI355X dense fp32 matrix
}  // namespace

void account(double bytes, double flops, bool same_launch) {
    add_to(g_bytes, bytes);
    add_to(g_flops, flops);
    const double tb = bytes / kHbmBytesPerS, tf = flops / kMfmaF32FlopPerS;
    add_to(g_ideal_s, tb > tf ? tb : tf);
    if (!same_launch) g_launches.fetch_add(1, std::memory_order_relaxed);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return CTAMD_OK;
    return fail(e == hipErrorOutOfMemory ? CTAMD_ENOMEM : CTAMD_EHIP, "%s: %s", what, hipGetErrorString(e));
}

int launched(const char* kernel) { return check_hip(hipGetLastError(), kernel); }

static int current_device() {
    int d = -1;
    if (hipGetDevice(&d) != hipSuccess) return -1;
    return d;
}

const float* pad_neg_inf() {
    float* s = scratch();
    return s ? s + kScratchFloats : nullptr;
}
const float* pad_zero() {
    float* s = scratch();
    return s ? s + kScratchFloats + 4 : nullptr;
}

namespace {
bool g_scratch_used[kMaxDevices] = {};
void* g_scratch_user[kMaxDevices] = {};      // the stream whose work used the scratch last (compared, never used)
bool g_user_blocking[kMaxDevices] = {};      // whether that stream orders itself with the null stream
bool g_event_recorded[kMaxDevices] = {};     // g_scratch_event marks the end of that stream's scratch-using work
hipEvent_t g_scratch_event[kMaxDevices] = {};
void* g_recording = nullptr;                 // the stream a graph is being recorded on, if any

bool blocking(void* stream) {                // orders itself with the null stream
    if (!stream || stream == g_recording) return true;   // recordings are made on streams of ctamd_stream_create
    unsigned flags = 0;
    if (hipStreamGetFlags(as_stream(stream), &flags) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return !(flags & hipStreamNonBlocking);
}
bool capturing(void* stream) {
    if (!stream) return false;
    if (stream == g_recording) return true;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(as_stream(stream), &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}
int scratch_event(int d, hipEvent_t* ev) {
    if (!g_scratch_event[d]) {
        int rc = check_hip(hipEventCreateWithFlags(&g_scratch_event[d], hipEventDisableTiming), "hipEventCreate(scratch)");
        if (rc) return rc;
    }
    *ev = g_scratch_event[d];
    return CTAMD_OK;
}
}  // namespace

int scratch_claim(void* stream) {
    int d = current_device();
    if (d < 0 || d >= kMaxDevices) return fail(CTAMD_EINVAL, "no current device");
    std::lock_guard<std::mutex> lock(g_mu);
    void* user = g_scratch_user[d];
    if (g_scratch_used[d] && user != stream) {
        if (user == g_recording && user)
            return fail(CTAMD_EINVAL, "the device scratch belongs to the graph being recorded on another stream");
        if (!capturing(stream)) {            // a recording runs nothing now; its replays claim the scratch themselves
            hipEvent_t ev = nullptr;
            if (!user) {
                // the null stream was the user: blocking streams follow it by themselves, any other waits
                // for an event recorded on it now (the null stream's handle cannot go stale)
                if (!blocking(stream)) {
                    int rc = scratch_event(d, &ev);
                    if (!rc) rc = check_hip(hipEventRecord(ev, nullptr), "hipEventRecord(scratch)");
                    if (!rc) rc = check_hip(hipStreamWaitEvent(as_stream(stream), ev, 0), "hipStreamWaitEvent(scratch)");
                    if (rc) return rc;
                }
            } else if (g_event_recorded[d] && !(stream == nullptr && g_user_blocking[d])) {
                int rc = scratch_event(d, &ev);
                if (!rc) rc = check_hip(hipStreamWaitEvent(as_stream(stream), ev, 0), "hipStreamWaitEvent(scratch)");
                if (rc) return rc;
            }
        }
    }
    g_scratch_used[d] = true;
    if (user != stream) {
        g_scratch_user[d] = stream;
        g_user_blocking[d] = blocking(stream);
        g_event_recorded[d] = false;
    }
    return CTAMD_OK;
}

void scratch_release(void* stream) {
    int d = current_device();
    if (d < 0 || d >= kMaxDevices) return;
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_scratch_user[d] != stream) return;          // another thread's stream took over in between
    g_event_recorded[d] = false;
    if (!stream || capturing(stream)) return;
    hipEvent_t ev = nullptr;
    if (scratch_event(d, &ev) != CTAMD_OK) return;
    if (hipEventRecord(ev, as_stream(stream)) == hipSuccess) g_event_recorded[d] = true;
    else (void)hipGetLastError();
}

float* scratch() {
    int d = current_device();
    if (d < 0 || d >= kMaxDevices || g_scratch[d] == nullptr) {
        fail(CTAMD_EINVAL, "ctamd_init() has not been called for the current device");
        return nullptr;
    }
    return g_scratch[d];
}

bool fast_math() { return g_math_mode.load(std::memory_order_relaxed) == CTAMD_MATH_FAST; }

int compute_units() {
    int d = current_device();
    return (d < 0 || d >= kMaxDevices) ? 0 : g_cus[d];
}

}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int ctamd_init(int device) {
    int n = ctamd_device_count();
    if (n <= 0) return fail(CTAMD_ENODEV, "ctamd_init: no HIP device visible");
    if (device < 0 || device >= n || device >= 16) return fail(CTAMD_EINVAL, "ctamd_init: device %d out of range", device);
    int rc = check_hip(hipSetDevice(device), "hipSetDevice");
    if (rc) return rc;
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_scratch[device]) return CTAMD_OK;
    hipDeviceProp_t prop;
    rc = check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    if (rc) return rc;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(CTAMD_ENODEV, "ctamd_init: device %d is %s; this library is built for gfx950 only", device,
                    prop.gcnArchName);
    g_cus[device] = prop.multiProcessorCount;
    void* p = nullptr;
    rc = check_hip(hipMalloc(&p, (kScratchFloats + 8) * sizeof(float)), "hipMalloc(scratch)");
    if (rc) return rc;
    const float inf = __builtin_huge_valf();
    const float pads[8] = {-inf, -inf, -inf, -inf, 0.0f, 0.0f, 0.0f, 0.0f};
    rc = check_hip(hipMemcpy(static_cast<float*>(p) + kScratchFloats, pads, sizeof(pads), hipMemcpyHostToDevice),
                   "hipMemcpy(pads)");
    if (rc) {
        (void)hipFree(p);
        return rc;
    }
    double* static_scratch = nullptr;
    rc = static_partials(&static_scratch);      // this device's address of the static partials array
    if (rc) {
        (void)hipFree(p);
        return rc;
    }
    g_scratch[device] = static_cast<float*>(p);
    return CTAMD_OK;
}

const char* ctamd_last_error(void) { return g_err; }
int ctamd_set_math_mode(int mode) {
    if (mode != CTAMD_MATH_FAST && mode != CTAMD_MATH_EXACT) return fail(CTAMD_EINVAL, "%s: unknown mode %d", __func__, mode);
    g_math_mode.store(mode, std::memory_order_relaxed);
    return CTAMD_OK;
}
int ctamd_math_mode(void) { return g_math_mode.load(std::memory_order_relaxed); }
void ctamd_counters_reset(void) {
    g_bytes.store(0.0);
    g_flops.store(0.0);
    g_ideal_s.store(0.0);
    g_launches.store(0);
}
void ctamd_counters_read(double* bytes, double* flops, double* roofline_seconds, uint64_t* launches) {
    if (bytes) *bytes = g_bytes.load();
    if (flops) *flops = g_flops.load();
    if (roofline_seconds) *roofline_seconds = g_ideal_s.load();
    if (launches) *launches = g_launches.load();
}

// ---- streams and recorded launch sequences (HIP graphs)
int ctamd_stream_create(void** stream) {
    if (!stream) return fail(CTAMD_EINVAL, "%s: null output", __func__);
    hipStream_t s = nullptr;
    int rc = check_hip(hipStreamCreate(&s), "hipStreamCreate");   // default priority, blocking w.r.t. the null stream
    *stream = rc ? nullptr : static_cast<void*>(s);
    return rc;
}
int ctamd_stream_destroy(void* stream) {
    if (!stream) return CTAMD_OK;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        for (int d = 0; d < kMaxDevices; ++d)
            if (g_scratch_user[d] == stream) { g_scratch_user[d] = nullptr; g_scratch_used[d] = false; }   // destroying waits for its work
    }
    return check_hip(hipStreamDestroy(as_stream(stream)), "hipStreamDestroy");
}
int ctamd_graph_begin(void* stream) {
    if (!stream) return fail(CTAMD_EINVAL, "%s: the null stream cannot record", __func__);
    // relaxed: host-side calls that are not stream work (an allocation by a pool that ran dry)
    // stay legal while recording
    int rc = check_hip(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed), "hipStreamBeginCapture");
    if (!rc) {
        std::lock_guard<std::mutex> lock(g_mu);
        g_recording = stream;
    }
    return rc;
}
int ctamd_graph_end(void* stream, void** graph_out) {
    if (!stream || !graph_out) return fail(CTAMD_EINVAL, "%s: null argument", __func__);
    *graph_out = nullptr;
    hipGraph_t g = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        if (g_recording == stream) g_recording = nullptr;
    }
    int rc = check_hip(hipStreamEndCapture(as_stream(stream), &g), "hipStreamEndCapture");
    if (rc) return rc;
    hipGraphExec_t exec = nullptr;
    rc = check_hip(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0), "hipGraphInstantiate");
    (void)hipGraphDestroy(g);
    if (rc) return rc;
    *graph_out = static_cast<void*>(exec);
    return CTAMD_OK;
}
int ctamd_graph_launch(void* graph, void* stream) {
    if (!graph) return fail(CTAMD_EINVAL, "%s: null graph", __func__);
    ScratchUse use(stream);                      // recorded reductions use the device scratch at replay
    if (!use.ptr()) return CTAMD_EINVAL;
    return check_hip(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), as_stream(stream)), "hipGraphLaunch");
}
int ctamd_graph_destroy(void* graph) {
    if (!graph) return CTAMD_OK;
    return check_hip(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)), "hipGraphExecDestroy");
}

const char* ctamd_version(void) { return "ctorch_amd 0.1 (gfx950)"; }

int ctamd_malloc(void** ptr, size_t bytes) {
    if (!ptr) return fail(CTAMD_EINVAL, "ctamd_malloc: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) return CTAMD_OK;
    return check_hip(hipMalloc(ptr, bytes), "hipMalloc");
}

int ctamd_free(void* ptr) {
    if (!ptr) return CTAMD_OK;
    return check_hip(hipFree(ptr), "hipFree");
}

static int copy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind, void* stream, const char* what) {
    if (bytes == 0) return CTAMD_OK;
    if (!dst || !src) return fail(CTAMD_EINVAL, "%s: null pointer", what);
    return check_hip(hipMemcpyAsync(dst, src, bytes, kind, as_stream(stream)), what);
}

int ctamd_memcpy_h2d(void* dst, const void* src_host, size_t bytes, void* stream) {
    return copy(dst, src_host, bytes, hipMemcpyHostToDevice, stream, "ctamd_memcpy_h2d");
}
int ctamd_memcpy_d2h(void* dst_host, const void* src, size_t bytes, void* stream) {
    return copy(dst_host, src, bytes, hipMemcpyDeviceToHost, stream, "ctamd_memcpy_d2h");
}
int ctamd_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
    return copy(dst, src, bytes, hipMemcpyDeviceToDevice, stream, "ctamd_memcpy_d2d");
}
int ctamd_sync(void* stream) { return check_hip(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize"); }

int ctamd_read_small(void* dst_host, const void* src, size_t bytes, void* stream) {
    if (bytes == 0) return CTAMD_OK;
    if (!dst_host || !src) return fail(CTAMD_EINVAL, "ctamd_read_small: null pointer");
    if (bytes > CTAMD_READ_SMALL_MAX) return fail(CTAMD_ERANGE, "ctamd_read_small: %zu bytes, at most %d", bytes, CTAMD_READ_SMALL_MAX);
    // one page-locked landing buffer per host thread, allocated on the thread's first read and kept
    thread_local void* landing = nullptr;
    if (!landing) {
        int rc = check_hip(hipHostMalloc(&landing, CTAMD_READ_SMALL_MAX, hipHostMallocDefault), "hipHostMalloc(landing buffer)");
        if (rc) { landing = nullptr; return rc; }
    }
    int rc = check_hip(hipMemcpyAsync(landing, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)), "ctamd_read_small");
    if (!rc) rc = check_hip(hipStreamSynchronize(as_stream(stream)), "ctamd_read_small: hipStreamSynchronize");
    if (!rc) memcpy(dst_host, landing, bytes);
    return rc;
}

}  // extern "C"
