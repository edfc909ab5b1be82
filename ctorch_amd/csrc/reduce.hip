// Reductions: sum, Dot, MSE, MAE, the divisor scan of Div's backward and the column sum that
// reduces the gradient of a row-broadcast operand.  HBM-bound streams: 128-bit loads, several
// independent fp32 accumulators per thread, a wave64 butterfly, an LDS stage across the waves of
// a block, then one block folds the per-block partials (held as doubles in the device scratch)
// in a fixed order, so results are deterministic for a given size.
#include <mutex>

#include "colsum_small.h"
#include "common.h"

// Per-block partials of ctamd_dot_static_f32, the entry point for callers that cannot allocate:
// 2048 doubles (16 KiB) that every GPU the library runs on holds until the process ends.  In host
// code this name is only a handle for hipGetSymbolAddress; the device address it yields (one per
// device) is what launches are given.
static __device__ __align__(256) double scratch_static[2048];

namespace ctamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kUnroll = 4;
constexpr unsigned kMaxBlocks = 2048;   // partials folded by one block: keep that fold short
static_assert(sizeof(scratch_static) == kMaxBlocks * sizeof(double), "one partial per block of the largest grid");

// Device address of scratch_static on each device, looked up once per device with that device current.
constexpr int kStaticMaxDevices = 16;
std::mutex g_static_mu;
double* g_static_partials[kStaticMaxDevices] = {};

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Sum over the block; valid in thread 0.
__device__ __forceinline__ double block_sum(double v) {
    __shared__ double s_part[kWaves];
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = v;
    __syncthreads();
    double t = 0.0;
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) t += s_part[w];
    }
    return t;
}

struct SumT { static constexpr int kIn = 1;
    __device__ static float term(float a, float) { return a; } };
struct DotT { static constexpr int kIn = 2;
    __device__ static float term(float a, float b) { return a * b; } };
struct SqT { static constexpr int kIn = 2;
    __device__ static float term(float a, float b) { float d = a - b; return d * d; } };
struct AbsT { static constexpr int kIn = 2;
    __device__ static float term(float a, float b) { return __builtin_fabsf(a - b); } };
struct TinyT { static constexpr int kIn = 1;
    __device__ static float term(float a, float) { return (__builtin_fabsf(a) < 1.1920928955078125e-07f) ? 1.0f : 0.0f; } };

// Block b walks runs of kThreads*kUnroll consecutive vectors (b, b + gridDim, ...); within a run
// thread t takes vectors t, t+256, t+512, t+768, all loads issued before the first add.  The
// loads carry the non-temporal hint: every byte is used once.
template <class T, bool VEC>
__global__ __launch_bounds__(kThreads) void reduce_stage1(const float* __restrict__ a, const float* __restrict__ b,
                                                          double* __restrict__ partials, size_t n) {
    float acc[kUnroll][4];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[u][e] = 0.0f;
    float tail = 0.0f;
    if (VEC) {
        const size_t n4 = n >> 2;
        constexpr size_t kRun = size_t(kThreads) * kUnroll;
        for (size_t run = size_t(blockIdx.x) * kRun; run < n4; run += size_t(gridDim.x) * kRun) {
            v4f va[kUnroll], vb[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                size_t i = run + size_t(u) * kThreads + threadIdx.x;
                if (i < n4) {
                    va[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(a) + i);
                    if (T::kIn == 2) vb[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(b) + i);
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                size_t i = run + size_t(u) * kThreads + threadIdx.x;
                if (i < n4) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[u][e] += T::term(va[u][e], T::kIn == 2 ? vb[u][e] : 0.0f);
                }
            }
        }
        if (blockIdx.x == 0) {
            size_t i = (n4 << 2) + threadIdx.x;
            if (i < n) tail = T::term(a[i], T::kIn == 2 ? b[i] : 0.0f);
        }
    } else {
        const size_t tid = size_t(blockIdx.x) * kThreads + threadIdx.x;
        const size_t stride = size_t(gridDim.x) * kThreads;
        for (size_t i = tid; i < n; i += stride) acc[0][0] += T::term(a[i], T::kIn == 2 ? b[i] : 0.0f);
    }
    // pairwise fold of the 16 lanes, in double from here on
    double t = double(tail);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) t += (double(acc[u][0]) + double(acc[u][1])) + (double(acc[u][2]) + double(acc[u][3]));
    t = block_sum(t);
    if (threadIdx.x == 0) partials[blockIdx.x] = t;
}

// mode 0: out = float(total); 1: out = float(total) / float(n) (the reference divides the fp32
// sum by the element count converted to float); 2: flag = total > 0.
__global__ __launch_bounds__(kThreads) void reduce_stage2(const double* __restrict__ partials, unsigned count,
                                                          float* __restrict__ out, int32_t* __restrict__ flag,
                                                          int mode, float fn) {
    double t = 0.0;
    for (unsigned i = threadIdx.x; i < count; i += kThreads) t += partials[i];
    t = block_sum(t);
    if (threadIdx.x == 0) {
        if (mode == 0) out[0] = float(t);
        else if (mode == 1) out[0] = float(t) / fn;
        else flag[0] = (t > 0.0) ? 1 : 0;
    }
}

// `partials`: room for kMaxBlocks doubles in device memory (nullptr: the per-device scratch).
template <class T>
int reduce(const char* name, const float* a, const float* b, float* out, int32_t* flag, size_t n, int mode,
           void* stream, double* partials = nullptr) {
    if ((mode != 2 && !out) || (mode == 2 && !flag)) return fail(CTAMD_EINVAL, "%s: null output", name);
    if (n && (!a || (T::kIn == 2 && !b))) return fail(CTAMD_EINVAL, "%s: null input", name);
    ScratchUse use(stream, partials == nullptr);
    if (!partials) partials = reinterpret_cast<double*>(use.ptr());
    if (!partials) return CTAMD_EINVAL;
    hipStream_t s = as_stream(stream);
    unsigned grid = 0;
    if (n) {
        bool vec = aligned16(a) && (T::kIn == 1 || aligned16(b));
        size_t need = ((vec ? n / 4 + 1 : n) + size_t(kThreads) * kUnroll - 1) / (size_t(kThreads) * kUnroll);
        grid = need < kMaxBlocks ? unsigned(need) : kMaxBlocks;
        if (vec)
            hipLaunchKernelGGL((reduce_stage1<T, true>), dim3(grid), dim3(kThreads), 0, s, a, b, partials, n);
        else
            hipLaunchKernelGGL((reduce_stage1<T, false>), dim3(grid), dim3(kThreads), 0, s, a, b, partials, n);
        int rc = launched(name);
        if (rc) return rc;
    }
    hipLaunchKernelGGL(reduce_stage2, dim3(1), dim3(kThreads), 0, s, partials, grid, out, flag, mode, float(n));
    account(double(T::kIn) * 4.0 * double(n), T::kIn == 2 ? 2.0 * double(n) : double(n));
    return launched(name);
}

// ----------------------------------------------------------------------------- column sum
// A block owns a strip of 256 * CU vectors of columns (CU = 4: up to 4096 columns, 16 KiB per row;
// CU = 1 when that would leave the chip short of blocks) and a chunk of rows, and walks its rows in
// order, two (CU = 4) or four (CU = 1) rows in flight per thread.  Each block writes one partial row per strip; stage 2 adds
// the (at most 256) partial rows in double, four lanes per column with eight loads in flight each -
// a serial walk over the partial rows by one thread per column cost more than stage 1 itself.
template <bool VEC, int CU>
__global__ __launch_bounds__(kThreads) void colsum_stage1(const float* __restrict__ g, float* __restrict__ partials,
                                                          size_t rows, size_t cols, size_t rows_per_block) {
    constexpr int W = VEC ? 4 : 1;
    const size_t strip0 = size_t(blockIdx.x) * (size_t(kThreads) * CU * W);
    const size_t r0 = size_t(blockIdx.y) * rows_per_block;
    size_t r1 = r0 + rows_per_block;
    if (r1 > rows) r1 = rows;
    constexpr int P = CU == 1 ? 4 : 2;       // rows in flight per thread (P * CU loads)
    float acc[P][CU][4];
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
        for (int u = 0; u < CU; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[p][u][e] = 0.0f;
    size_t col[CU];
    bool live[CU];
#pragma unroll
    for (int u = 0; u < CU; ++u) {
        col[u] = strip0 + (size_t(u) * kThreads + threadIdx.x) * W;
        live[u] = col[u] < cols;
    }
    size_t r = r0;
    for (; r + (P - 1) < r1; r += P) {
        v4f x[P][CU];
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int u = 0; u < CU; ++u)
                if (live[u]) {
                    const float* src = g + (r + p) * cols + col[u];
                    if (VEC) x[p][u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src));
                    else x[p][u][0] = *src;
                }
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int u = 0; u < CU; ++u)
                if (live[u]) {
#pragma unroll
                    for (int e = 0; e < W; ++e) acc[p][u][e] += x[p][u][e];
                }
    }
    for (; r < r1; ++r) {
#pragma unroll
        for (int u = 0; u < CU; ++u)
            if (live[u]) {
                const float* src = g + r * cols + col[u];
                if (VEC) {
                    v4f x0 = *reinterpret_cast<const v4f*>(src);
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[0][u][e] += x0[e];
                } else {
                    acc[0][u][0] += *src;
                }
            }
    }
#pragma unroll
    for (int u = 0; u < CU; ++u)
        if (live[u]) {
#pragma unroll
            for (int e = 0; e < W; ++e) {
                float t = acc[0][u][e];
#pragma unroll
                for (int p = 1; p < P; ++p) t += acc[p][u][e];
                partials[size_t(blockIdx.y) * cols + col[u] + e] = t;
            }
        }
}

// Narrow matrices (a row is at most 128 vectors: the bias gradients of a layer, [8192 x 256] or
// [8192 x 10]): the strip kernel above would leave most of a block's threads without a column.  Here
// a block's threads form G = 256 / (vectors per row) row groups; group k walks rows k, k + G, ... of
// the block's chunk with four rows in flight, so the block reads its chunk as one contiguous run;
// the groups are added through LDS in group order and the block writes one partial row.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void colsum_narrow_stage1(const float* __restrict__ g, float* __restrict__ partials,
                                                                 size_t rows, size_t cols, unsigned lanes, unsigned groups,
                                                                 size_t rows_per_block) {
    __shared__ float s_part[kThreads * (VEC ? 4 : 1)];
    colsum_narrow_body<VEC>(g, partials, rows, cols, lanes, groups, rows_per_block, blockIdx.x, threadIdx.x, s_part);
}

static_assert(kColsumThreads == kThreads, "the shared body assumes this file's block size");
// out[c] = sum over the `chunks` rows of partials[., c], in double, LANES lanes per column.  Stage 2
// of the two-stage sum (LANES = 4), and the whole column sum of a small matrix (LANES = kSmallLanes,
// a bias gradient of a few hundred rows: one launch instead of two).
template <int LANES>
__global__ __launch_bounds__(kThreads) void colsum_stage2(const float* __restrict__ partials, float* __restrict__ out,
                                                          size_t cols, unsigned chunks) {
    __shared__ double s_acc[kThreads];
    colsum_fold_body<LANES>(partials, out, cols, chunks, blockIdx.x, threadIdx.x, s_acc);
}

}  // namespace

// The current device's copy of scratch_static: each GPU holds the array at its own address, so the
// lookup runs once per device with that device current (ctamd_init calls this; a first call of
// ctamd_dot_static_f32 on a device that was never initialised does as well).  Allocates nothing.
int static_partials(double** out) {
    *out = nullptr;
    int d = -1;
    int rc = check_hip(hipGetDevice(&d), "hipGetDevice");
    if (rc) return rc;
    if (d < 0 || d >= kStaticMaxDevices) return fail(CTAMD_EINVAL, "device %d out of range", d);
    std::lock_guard<std::mutex> lock(g_static_mu);
    if (!g_static_partials[d]) {
        void* p = nullptr;
        rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch_static)), "hipGetSymbolAddress(scratch_static)");
        if (rc) return rc;
        if (!p) return fail(CTAMD_EHIP, "hipGetSymbolAddress(scratch_static) returned no address");
        g_static_partials[d] = static_cast<double*>(p);
    }
    *out = g_static_partials[d];
    return CTAMD_OK;
}

}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_dot_static_f32(const float* a, const float* b, float* out, size_t n, void* s) {
    if (n > CTAMD_DOT_STATIC_MAX_N)
        return fail(CTAMD_ERANGE, "%s: %zu elements exceed the supported maximum of %zu", __func__, n,
                    size_t(CTAMD_DOT_STATIC_MAX_N));
    double* partials = nullptr;
    int rc = static_partials(&partials);
    if (rc) return rc;
    // every partial the fold launch reads was written by this call's first launch: nothing to clear
    return reduce<DotT>(__func__, a, b, out, nullptr, n, 0, s, partials);
}

int ctamd_sum_f32(const float* a, float* out, size_t n, void* s) { return reduce<SumT>(__func__, a, nullptr, out, nullptr, n, 0, s); }
int ctamd_dot_f32(const float* a, const float* b, float* out, size_t n, void* s) { return reduce<DotT>(__func__, a, b, out, nullptr, n, 0, s); }
int ctamd_mse_f32(const float* a, const float* b, float* out, size_t n, void* s) { return reduce<SqT>(__func__, a, b, out, nullptr, n, 1, s); }
int ctamd_mae_f32(const float* a, const float* b, float* out, size_t n, void* s) { return reduce<AbsT>(__func__, a, b, out, nullptr, n, 1, s); }
int ctamd_any_abs_lt_eps_f32(const float* b, int32_t* flag, size_t n, void* s) {
    return reduce<TinyT>(__func__, b, nullptr, nullptr, flag, n, 2, s);
}

int ctamd_colsum_f32(const float* g, float* out, size_t rows, size_t cols, void* stream) {
    if (cols == 0) return CTAMD_OK;
    if (!out) return fail(CTAMD_EINVAL, "%s: null output", __func__);
    if (rows == 0) return ctamd_fill_f32(out, 0.0f, cols, stream);
    if (!g) return fail(CTAMD_EINVAL, "%s: null input", __func__);
    if (rows > (size_t(1) << 62) / cols) return fail(CTAMD_ERANGE, "%s: rows*cols overflows", __func__);
    hipStream_t s = as_stream(stream);
    if (colsum_is_small(rows, cols)) {                            // one launch, rows added in order
        hipLaunchKernelGGL(colsum_stage2<kSmallLanes>, dim3(colsum_small_blocks(cols)), dim3(kThreads), 0, s, g, out,
                           cols, (unsigned)rows);
        account(4.0 * double(rows) * double(cols), double(rows) * double(cols));
        return launched(__func__);
    }
    ScratchUse use(stream);
    float* partials = use.ptr();
    if (!partials) return CTAMD_EINVAL;
    if (cols > kScratchFloats) return fail(CTAMD_ERANGE, "%s: more than %zu columns", __func__, kScratchFloats);
    bool vec = (cols % 4 == 0) && aligned16(g);
    const size_t w = vec ? 4 : 1;
    const size_t cus = size_t(compute_units() > 0 ? compute_units() : 256);
    ColsumNarrowPlan narrow;
    if (colsum_narrow_plan(rows, cols, vec, &narrow)) {
        const size_t lanes = narrow.lanes, groups = narrow.groups, rows_per_block = narrow.rows_per_block, chunks = narrow.chunks;
        if (vec)
            hipLaunchKernelGGL((colsum_narrow_stage1<true>), dim3((unsigned)chunks), dim3(kThreads), 0, s, g, partials, rows, cols,
                               (unsigned)lanes, (unsigned)groups, rows_per_block);
        else
            hipLaunchKernelGGL((colsum_narrow_stage1<false>), dim3((unsigned)chunks), dim3(kThreads), 0, s, g, partials, rows, cols,
                               (unsigned)lanes, (unsigned)groups, rows_per_block);
        int rc = launched(__func__);
        if (rc) return rc;
        constexpr size_t kFoldCols = kThreads / kFoldLanes;
        hipLaunchKernelGGL(colsum_stage2<kFoldLanes>, dim3((unsigned)((cols + kFoldCols - 1) / kFoldCols)), dim3(kThreads), 0, s,
                           partials, out, cols, (unsigned)chunks);
        account(4.0 * double(rows) * double(cols), double(rows) * double(cols));
        return launched(__func__);
    }
    // at most 256 row chunks of at least 16 rows; wide strips unless that leaves the chip short of blocks
    size_t chunks = (rows + 15) / 16;
    if (chunks > 256) chunks = 256;
    if (chunks > kScratchFloats / cols) chunks = kScratchFloats / cols;
    if (chunks < 1) chunks = 1;
    size_t rows_per_block = (rows + chunks - 1) / chunks;
    chunks = (rows + rows_per_block - 1) / rows_per_block;
    const size_t wide_strips = (cols + size_t(kThreads) * 4 * w - 1) / (size_t(kThreads) * 4 * w);
    const bool wide = wide_strips * chunks >= 4 * cus;
    const size_t strip = size_t(kThreads) * (wide ? 4 : 1) * w;
    size_t col_blocks = (cols + strip - 1) / strip;
    if (col_blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: too many columns", __func__);
    dim3 grid((unsigned)col_blocks, (unsigned)chunks);
    if (vec && wide)
        hipLaunchKernelGGL((colsum_stage1<true, 4>), grid, dim3(kThreads), 0, s, g, partials, rows, cols, rows_per_block);
    else if (vec)
        hipLaunchKernelGGL((colsum_stage1<true, 1>), grid, dim3(kThreads), 0, s, g, partials, rows, cols, rows_per_block);
    else if (wide)
        hipLaunchKernelGGL((colsum_stage1<false, 4>), grid, dim3(kThreads), 0, s, g, partials, rows, cols, rows_per_block);
    else
        hipLaunchKernelGGL((colsum_stage1<false, 1>), grid, dim3(kThreads), 0, s, g, partials, rows, cols, rows_per_block);
    int rc = launched(__func__);
    if (rc) return rc;
    constexpr size_t kFoldCols = kThreads / kFoldLanes;
    hipLaunchKernelGGL(colsum_stage2<kFoldLanes>, dim3((unsigned)((cols + kFoldCols - 1) / kFoldCols)), dim3(kThreads), 0, s, partials,
                       out, cols, (unsigned)chunks);
    account(4.0 * double(rows) * double(cols), double(rows) * double(cols));
    return launched(__func__);
}

}  // extern "C"
