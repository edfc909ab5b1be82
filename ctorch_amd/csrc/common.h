// Shared plumbing of the launch layer: error reporting, argument checks, launch geometry and the
// per-device reduction scratch.
#ifndef CTORCH_AMD_COMMON_H
#define CTORCH_AMD_COMMON_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/ctorch_amd.h"

namespace ctamd {

// Records the message returned by ctamd_last_error() and passes `code` through.
int fail(int code, const char* fmt, ...);
// Maps a hipError_t to 0 / CTAMD_EHIP, recording where it happened.
int check_hip(hipError_t e, const char* what);
// Checks the error state after a kernel launch.
int launched(const char* kernel);

// Scratch for two-stage reductions: kScratchFloats fp32 slots per device, allocated by
// ctamd_init() and never freed.  Returns nullptr (and records an error) before ctamd_init().
constexpr size_t kScratchFloats = size_t(1) << 24;   // 64 MiB
float* scratch();
// The scratch for work about to be launched on `stream`.  One buffer serves every stream of a device, so
// its users are put in order: a stream other than the previous user first waits (on the device,
// hipStreamWaitEvent) for the point the previous user had reached when it finished its own
// scratch-using launches.  That point is an event owned by the library, recorded by release() on the
// stream the caller has just passed in - a stream handle kept from an earlier call is never touched
// again, it may have been destroyed by its owner since.  The null stream needs no event per use (one
// is recorded on it when another stream takes over; blocking streams order themselves with it
// anyway).  A stream that is recording a graph waits for nothing and records nothing: its launches
// run at replay, and replays claim the scratch through ctamd_graph_launch.
// Use: `ScratchUse use(stream); float* p = use.ptr(); if (!p) return CTAMD_EINVAL; ...launches...`;
// the destructor releases after the last launch of the scope.
int scratch_claim(void* stream);
void scratch_release(void* stream);
class ScratchUse {
  public:
    explicit ScratchUse(void* stream, bool wanted = true) : stream_(stream), held_(false), ptr_(nullptr) {
        if (wanted) acquire();
    }
    ~ScratchUse() {
        if (held_) scratch_release(stream_);
    }
    ScratchUse(const ScratchUse&) = delete;
    ScratchUse& operator=(const ScratchUse&) = delete;
    // claims now (for scopes that learn late whether they need the scratch); nullptr on failure
    float* acquire() {
        if (!held_) {
            float* s = scratch();
            if (s && scratch_claim(stream_) == CTAMD_OK) {
                held_ = true;
                ptr_ = s;
            }
        }
        return ptr_;
    }
    float* ptr() const { return ptr_; }

  private:
    void* stream_;
    bool held_;
    float* ptr_;
};
// Four floats of -inf / of 0 in device memory (set up by ctamd_init): what row kernels read in
// place of a vector that would lie beyond the end of a row.
const float* pad_neg_inf();
const float* pad_zero();
// Looks up (once per device) the current device's address of the static partials array that
// ctamd_dot_static_f32 uses; defined in reduce.hip next to the array.
int static_partials(double** out);
// Whether softmax, the cross-entropy gradients and fused expressions evaluate their transcendentals in
// single precision (<= 2 ulp, the default) or with the double-precision routines that return glibc's
// floats bit for bit; set by ctamd_set_math_mode().
bool fast_math();
// Compute units of the current device (256 on MI355X); 0 before ctamd_init().
int compute_units();

// Adds one operator launch to the per-process work counters read by ctamd_counters_read():
// `bytes` and `flops` are the operator's algorithmic traffic and arithmetic (what it must move and
// compute, not what the kernels happen to do).
// same_launch: work that rides in a launch already counted (the count of launches stays).
void account(double bytes, double flops, bool same_launch = false);

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

// A class index kept as a float, read the way the reference reads it (a conversion to int that truncates
// toward zero).  NaN: the reference's host turns it into the most negative int, which no class count
// admits; the conversion instruction here would make it 0, a valid class - so it is mapped out of range.
// Infinities and magnitudes beyond int saturate on this side and are out of range on both.
__device__ __forceinline__ int class_index(float t) { return t == t ? int(t) : -1; }

// Grid for a streaming kernel: enough 256-thread blocks to cover `work_items` (each block
// iteration handles `per_block` items), capped at `waves_per_cu`-deep occupancy of the chip so
// that grid-stride loops amortise launch cost on large tensors.
inline unsigned stream_grid(size_t work_items, size_t per_block, int blocks_per_cu = 8) {
    size_t need = (work_items + per_block - 1) / per_block;
    size_t cap = size_t(compute_units() > 0 ? compute_units() : 256) * size_t(blocks_per_cu);
    if (need < 1) need = 1;
    return unsigned(need < cap ? need : cap);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// A result of at most this many bytes - a quarter of the 256 MiB memory-side cache - is stored
// without the streaming hint by the elementwise kernels: what reads it next finds it in that cache,
// and a buffer that is overwritten before it was evicted never costs HBM a write (the 28 launches of
// a forward and backward pass over 64 MiB tensors: 851 -> 822 us).  Measured at 256 MiB per tensor,
// one input: a chain in which every launch reads the result of the one before runs 78 us per launch
// with hinted loads and plain stores against 85 us with the hint on both sides, but launches over
// unrelated buffers lose (88 against 84 us; a kernel that re-reads its input, like the column
// softmax, 161 against 139 us: the result pushes the input out), and at 1 GiB per tensor the hint
// on both sides wins too (352 against 365 us).  Hence the bound well below the cache size.
// The choice has to be a template argument of the kernel: a hinted and a plain store on the two
// sides of a branch are folded by the compiler into ONE plain store.
constexpr size_t kResidentBytes = size_t(64) << 20;
inline bool result_streams(size_t bytes) { return bytes > kResidentBytes; }

}  // namespace ctamd

#define CTAMD_REQUIRE(cond, msg)                                                 \
    do {                                                                         \
        if (!(cond)) return ::ctamd::fail(CTAMD_EINVAL, "%s: %s", __func__, msg); \
    } while (0)

#endif
