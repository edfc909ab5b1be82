// Reductions: sum, Dot, MSE, MAE, the divisor scan of Div's backward and the column sum that
// reduces the gradient of a row-broadcast operand.  HBM-bound streams: 128-bit loads, several
// independent fp32 accumulators per thread, a wave64 butterfly, an LDS stage across the waves of
// a block, then one block folds the per-block partials (held as doubles in the device scratch)
// in a fixed order, so results are deterministic for a given size.
#include "common.h"

namespace ctamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kUnroll = 4;
constexpr unsigned kMaxBlocks = 2048;   // partials folded by one block: keep that fold short

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

template <class T>
int reduce(const char* name, const float* a, const float* b, float* out, int32_t* flag, size_t n, int mode,
           void* stream) {
    if ((mode != 2 && !out) || (mode == 2 && !flag)) return fail(CTAMD_EINVAL, "%s: null output", name);
    if (n && (!a || (T::kIn == 2 && !b))) return fail(CTAMD_EINVAL, "%s: null input", name);
    double* partials = reinterpret_cast<double*>(scratch());
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
    return launched(name);
}

// ----------------------------------------------------------------------------- column sum
// Block = 64 column groups x 4 row lanes.  Each block folds a chunk of rows for its columns and
// writes one partial row; stage 2 adds the partial rows in double.
constexpr int kColLanes = 64;
constexpr int kRowLanes = 4;

template <bool VEC>
__global__ __launch_bounds__(kThreads) void colsum_stage1(const float* __restrict__ g, float* __restrict__ partials,
                                                          size_t rows, size_t cols, size_t rows_per_block) {
    constexpr int W = VEC ? 4 : 1;
    const int tx = threadIdx.x % kColLanes, ty = threadIdx.x / kColLanes;
    const size_t col = (size_t(blockIdx.x) * kColLanes + tx) * W;
    const size_t r0 = size_t(blockIdx.y) * rows_per_block;
    size_t r1 = r0 + rows_per_block;
    if (r1 > rows) r1 = rows;
    constexpr int U = 8;    // independent row loads in flight per thread
    float acc[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    if (col < cols) {
        size_t r = r0 + ty;
        for (; r + size_t(U - 1) * kRowLanes < r1; r += size_t(U) * kRowLanes) {
            if (VEC) {
                v4f x[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    x[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(g + (r + size_t(u) * kRowLanes) * cols + col));
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[u & 1][e] += x[u][e];
            } else {
                float x[U];
#pragma unroll
                for (int u = 0; u < U; ++u) x[u] = g[(r + size_t(u) * kRowLanes) * cols + col];
#pragma unroll
                for (int u = 0; u < U; ++u) acc[u & 1][0] += x[u];
            }
        }
        for (; r < r1; r += kRowLanes) {
            if (VEC) {
                v4f x0 = *reinterpret_cast<const v4f*>(g + r * cols + col);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[0][e] += x0[e];
            } else {
                acc[0][0] += g[r * cols + col];
            }
        }
    }
    __shared__ float s_acc[kRowLanes][kColLanes][4];
#pragma unroll
    for (int e = 0; e < W; ++e) s_acc[ty][tx][e] = acc[0][e] + acc[1][e];
    __syncthreads();
    if (ty == 0 && col < cols) {
#pragma unroll
        for (int e = 0; e < W; ++e) {
            float t = (s_acc[0][tx][e] + s_acc[1][tx][e]) + (s_acc[2][tx][e] + s_acc[3][tx][e]);
            partials[size_t(blockIdx.y) * cols + col + e] = t;
        }
    }
}

__global__ __launch_bounds__(kThreads) void colsum_stage2(const float* __restrict__ partials, float* __restrict__ out,
                                                          size_t cols, unsigned chunks) {
    size_t c = size_t(blockIdx.x) * kThreads + threadIdx.x;
    if (c >= cols) return;
    double t = 0.0;
    for (unsigned k = 0; k < chunks; ++k) t += double(partials[size_t(k) * cols + c]);
    out[c] = float(t);
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" {

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
    float* partials = scratch();
    if (!partials) return CTAMD_EINVAL;
    if (cols > kScratchFloats) return fail(CTAMD_ERANGE, "%s: more than %zu columns", __func__, kScratchFloats);
    bool vec = (cols % 4 == 0) && aligned16(g);
    size_t col_blocks = (cols + size_t(kColLanes) * (vec ? 4 : 1) - 1) / (size_t(kColLanes) * (vec ? 4 : 1));
    // row chunks: fill the chip (about 8 blocks per CU), at least 32 rows per block, and the
    // partial rows must fit the scratch
    size_t want = (size_t(compute_units() > 0 ? compute_units() : 256) * 8 + col_blocks - 1) / col_blocks;
    size_t chunks = (rows + 63) / 64;
    if (chunks > want) chunks = want;
    if (chunks > kScratchFloats / cols) chunks = kScratchFloats / cols;
    if (chunks > 65535) chunks = 65535;
    if (chunks < 1) chunks = 1;
    size_t rows_per_block = (rows + chunks - 1) / chunks;
    chunks = (rows + rows_per_block - 1) / rows_per_block;
    hipStream_t s = as_stream(stream);
    dim3 grid((unsigned)col_blocks, (unsigned)chunks);
    if (col_blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: too many columns", __func__);
    if (vec)
        hipLaunchKernelGGL((colsum_stage1<true>), grid, dim3(kThreads), 0, s, g, partials, rows, cols, rows_per_block);
    else
        hipLaunchKernelGGL((colsum_stage1<false>), grid, dim3(kThreads), 0, s, g, partials, rows, cols, rows_per_block);
    int rc = launched(__func__);
    if (rc) return rc;
    hipLaunchKernelGGL(colsum_stage2, dim3((unsigned)((cols + kThreads - 1) / kThreads)), dim3(kThreads), 0, s, partials,
                       out, cols, (unsigned)chunks);
    return launched(__func__);
}

}  // extern "C"
