// Row softmax, cross entropy (one-hot and class-index targets) and their gradients.
//
// One block owns one row at a time and keeps the whole row in registers, so the logits are read
// from HBM exactly once: max, exp(x - max), the row sum and the normalisation all run on the
// resident copy (one wave64 butterfly plus an LDS stage across waves per reduction).  Rows longer
// than a block can hold (more than 32768 columns, or more than 8192 when the row is not
// 16-byte aligned) take a streaming variant that walks the row with an online (max, sum) pair
// and reads it a second time to normalise.  exp() is devmath.h's, bit-identical to the
// reference's libm call, so each exp(x - max) equals the reference's; only the order of the row
// sum differs (tree instead of sequential).  Compile with -ffp-contract=off.
#include <math.h>

#include "common.h"
#include "devmath.h"

namespace ctamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float o = __shfl_xor(v, off, 64);
        v = (o > v) ? o : v;
    }
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Block-wide reductions whose result every thread receives.  `slot` is LDS of THREADS/64 + 1
// entries; consecutive calls must use distinct slots or be separated by the caller's barrier -
// each call ends with the barrier that makes its slot reusable two calls later.
template <int THREADS, class V, class Fold>
__device__ __forceinline__ V block_all(V v, V* slot, Fold fold) {
    if (THREADS == 64) return v;
    constexpr int W = THREADS / 64;
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    V t = slot[0];
#pragma unroll
    for (int w = 1; w < W; ++w) t = fold(t, slot[w]);
    __syncthreads();
    return t;
}
template <int THREADS>
__device__ __forceinline__ float block_max(float v, float* slot) {
    return block_all<THREADS>(wave_max(v), slot, [](float a, float b) { return (b > a) ? b : a; });
}
template <int THREADS>
__device__ __forceinline__ float block_sum(float v, float* slot) {
    return block_all<THREADS>(wave_sum(v), slot, [](float a, float b) { return a + b; });
}
template <int THREADS>
__device__ __forceinline__ double block_sum(double v, double* slot) {
    return block_all<THREADS>(wave_sum(v), slot, [](double a, double b) { return a + b; });
}

__device__ __forceinline__ void stage_exp_table(uint64_t* exp2) {
    if (threadIdx.x < 32) exp2[threadIdx.x] = cta_exp2_tab[threadIdx.x];
    __syncthreads();
}

constexpr float kNegInf = -__builtin_huge_valf();

// A row held in registers: ITEMS groups of W floats per thread, group k of thread t covering
// elements [(t + k*THREADS) * W, +W).
template <int THREADS, int ITEMS, int W>
struct Row {
    float v[ITEMS][W];
    __device__ __forceinline__ void load(const float* __restrict__ p, size_t cols, float pad) {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            size_t e = (size_t(threadIdx.x) + size_t(k) * THREADS) * W;
            if (e < cols) {
                if (W == 4) {
                    v4f t = *reinterpret_cast<const v4f*>(p + e);
#pragma unroll
                    for (int i = 0; i < W; ++i) v[k][i] = t[i];
                } else {
                    v[k][0] = p[e];
                }
            } else {
#pragma unroll
                for (int i = 0; i < W; ++i) v[k][i] = pad;
            }
        }
    }
    __device__ __forceinline__ void store(float* __restrict__ p, size_t cols) const {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            size_t e = (size_t(threadIdx.x) + size_t(k) * THREADS) * W;
            if (e < cols) {
                if (W == 4) {
                    v4f t;
#pragma unroll
                    for (int i = 0; i < W; ++i) t[i] = v[k][i];
                    *reinterpret_cast<v4f*>(p + e) = t;
                } else {
                    p[e] = v[k][0];
                }
            }
        }
    }
    __device__ __forceinline__ float max() const {
        float m = kNegInf;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
#pragma unroll
            for (int i = 0; i < W; ++i) m = (v[k][i] > m) ? v[k][i] : m;
        return m;
    }
    // v <- exp(v - m) (padding lanes hold -inf and give exactly 0); returns this thread's sum
    __device__ __forceinline__ float exp_shifted(float m, const uint64_t* exp2) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
#pragma unroll
            for (int i = 0; i < W; ++i) {
                v[k][i] = cta_expf_tab(v[k][i] - m, exp2);
                s += v[k][i];
            }
        return s;
    }
    __device__ __forceinline__ size_t index(int k, int i) const {
        return (size_t(threadIdx.x) + size_t(k) * THREADS) * W + i;
    }
};

enum Mode { kSoftmax, kCeOnehot, kCeIndex, kCeBwdOnehot, kCeBwdIndex, kSoftmaxBwd };

struct Args {
    const float* x;      // logits / softmax output y (kSoftmaxBwd)
    const float* t;      // one-hot targets / class indices / upstream gradient (kSoftmaxBwd)
    const float* g1;     // 0-D upstream gradient of the loss (backward modes)
    float* out;          // y / dx
    double* partials;    // per-block loss partials (forward loss modes)
    int32_t* status;     // bad-index flag (kCeIndex), may be null
    size_t rows, cols;
};

template <int MODE, int THREADS, int ITEMS, int W>
__global__ __launch_bounds__(THREADS) void row_kernel(Args a) {
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_f[2][THREADS / 64 + 1];
    __shared__ double s_d[THREADS / 64 + 1];
    stage_exp_table(s_exp2);
    double block_loss = 0.0;
    for (size_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const float* xr = a.x + row * a.cols;
        Row<THREADS, ITEMS, W> r;
        if (MODE == kSoftmaxBwd) {
            // r = y, q = g: d = sum g*y, dx = y * (g - d)
            Row<THREADS, ITEMS, W> q;
            r.load(xr, a.cols, 0.0f);
            q.load(a.t + row * a.cols, a.cols, 0.0f);
            float d = 0.0f;
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) d += q.v[k][i] * r.v[k][i];
            d = block_sum<THREADS>(d, s_f[0]);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) r.v[k][i] = r.v[k][i] * (q.v[k][i] - d);
            r.store(a.out + row * a.cols, a.cols);
            continue;
        }
        r.load(xr, a.cols, kNegInf);
        const float m = block_max<THREADS>(r.max(), s_f[0]);
        const float s = block_sum<THREADS>(r.exp_shifted(m, s_exp2), s_f[1]);
        if (MODE == kSoftmax) {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) r.v[k][i] = r.v[k][i] / s;
            r.store(a.out + row * a.cols, a.cols);
        } else if (MODE == kCeOnehot) {
            // -sum_j t_j * log(max(e_j / s, 1e-10)); terms with t_j == 0 contribute exactly 0
            Row<THREADS, ITEMS, W> q;
            q.load(a.t + row * a.cols, a.cols, 0.0f);
            double loss = 0.0;
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    float tj = q.v[k][i];
                    if (tj != 0.0f) {
                        float p = r.v[k][i] / s;
                        p = (p < 1e-10f) ? 1e-10f : p;
                        float lg = float(log(double(p)));
                        loss -= double(tj * lg);
                    }
                }
            loss = block_sum<THREADS>(loss, s_d);
            block_loss += loss;
        } else if (MODE == kCeIndex) {
            const int c = int(a.t[row]);
            if (c < 0 || c >= int(a.cols)) {
                if (threadIdx.x == 0 && a.status) a.status[0] = 1;
                block_loss += double(__builtin_nanf(""));
            } else {
                // the thread that holds column c publishes exp(x_c - m)
                float ec = 0.0f;
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                    for (int i = 0; i < W; ++i)
                        if (r.index(k, i) == size_t(c)) ec = r.v[k][i];
                ec = block_sum<THREADS>(ec, s_f[0]);
                float p = ec / s;
                p = (p < 1e-10f) ? 1e-10f : p;
                block_loss -= double(float(log(double(p))));
            }
        } else {   // kCeBwdOnehot / kCeBwdIndex: dx = (e / s - t) * g
            const float g = a.g1[0];
            if (MODE == kCeBwdOnehot) {
                Row<THREADS, ITEMS, W> q;
                q.load(a.t + row * a.cols, a.cols, 0.0f);
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                    for (int i = 0; i < W; ++i) {
                        float sm = r.v[k][i] / s;
                        float d = sm - q.v[k][i];
                        r.v[k][i] = d * g;
                    }
            } else {
                const int c = int(a.t[row]);
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                    for (int i = 0; i < W; ++i) {
                        float sm = r.v[k][i] / s;
                        float d = sm - ((r.index(k, i) == size_t(c) && c >= 0) ? 1.0f : 0.0f);
                        r.v[k][i] = d * g;
                    }
            }
            r.store(a.out + row * a.cols, a.cols);
        }
    }
    if ((MODE == kCeOnehot || MODE == kCeIndex) && threadIdx.x == 0) a.partials[blockIdx.x] = block_loss;
}

// Streaming variant for rows that do not fit a block's registers: pass 1 keeps an online
// (max, sum) pair per thread - sum is rescaled by exp(old_max - new_max) whenever the max grows -
// pass 2 re-reads the row.  The rescaled sum differs from sum(exp(x - max)) by rounding only.
template <int MODE>
__global__ __launch_bounds__(1024) void row_stream_kernel(Args a) {
    constexpr int THREADS = 1024;
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_f[2][THREADS / 64 + 1];
    __shared__ double s_d[THREADS / 64 + 1];
    stage_exp_table(s_exp2);
    double block_loss = 0.0;
    for (size_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const float* xr = a.x + row * a.cols;
        if (MODE == kSoftmaxBwd) {
            const float* gr = a.t + row * a.cols;
            float d = 0.0f;
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) d += gr[j] * xr[j];
            d = block_sum<THREADS>(d, s_f[0]);
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) a.out[row * a.cols + j] = xr[j] * (gr[j] - d);
            continue;
        }
        float m = kNegInf, s = 0.0f;
        for (size_t j = threadIdx.x; j < a.cols; j += THREADS) {
            float v = xr[j];
            if (v > m) {
                s = s * cta_expf_tab(m - v, s_exp2);
                m = v;
            }
            s += cta_expf_tab(v - m, s_exp2);
        }
        const float M = block_max<THREADS>(m, s_f[0]);
        s = (m == kNegInf) ? 0.0f : s * cta_expf_tab(m - M, s_exp2);
        const float S = block_sum<THREADS>(s, s_f[1]);
        if (MODE == kSoftmax) {
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS)
                a.out[row * a.cols + j] = cta_expf_tab(xr[j] - M, s_exp2) / S;
        } else if (MODE == kCeOnehot) {
            const float* tr = a.t + row * a.cols;
            double loss = 0.0;
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) {
                float tj = tr[j];
                if (tj != 0.0f) {
                    float p = cta_expf_tab(xr[j] - M, s_exp2) / S;
                    p = (p < 1e-10f) ? 1e-10f : p;
                    loss -= double(tj * float(log(double(p))));
                }
            }
            block_loss += block_sum<THREADS>(loss, s_d);
        } else if (MODE == kCeIndex) {
            const int c = int(a.t[row]);
            if (c < 0 || c >= int(a.cols)) {
                if (threadIdx.x == 0 && a.status) a.status[0] = 1;
                block_loss += double(__builtin_nanf(""));
            } else {
                float p = cta_expf_tab(xr[c] - M, s_exp2) / S;
                p = (p < 1e-10f) ? 1e-10f : p;
                block_loss -= double(float(log(double(p))));
            }
        } else {
            const float g = a.g1[0];
            const int c = (MODE == kCeBwdIndex) ? int(a.t[row]) : -1;
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) {
                float sm = cta_expf_tab(xr[j] - M, s_exp2) / S;
                float tj = (MODE == kCeBwdOnehot) ? a.t[row * a.cols + j] : ((j == size_t(c) && c >= 0) ? 1.0f : 0.0f);
                float d = sm - tj;
                a.out[row * a.cols + j] = d * g;
            }
        }
    }
    if ((MODE == kCeOnehot || MODE == kCeIndex) && threadIdx.x == 0) a.partials[blockIdx.x] = block_loss;
}

// out[0] = float(sum of partials), folded in a fixed order.
__global__ __launch_bounds__(256) void loss_stage2(const double* __restrict__ partials, unsigned count,
                                                   float* __restrict__ out) {
    __shared__ double s_d[256 / 64 + 1];
    double t = 0.0;
    for (unsigned i = threadIdx.x; i < count; i += 256) t += partials[i];
    t = block_sum<256>(t, s_d);
    if (threadIdx.x == 0) out[0] = float(t);
}

__global__ void clear_i32(int32_t* p) { p[0] = 0; }

constexpr unsigned kMaxRowBlocks = 1u << 16;

template <int MODE, int THREADS, int ITEMS, int W>
void launch_cfg(const Args& a, unsigned grid, hipStream_t s) {
    hipLaunchKernelGGL((row_kernel<MODE, THREADS, ITEMS, W>), dim3(grid), dim3(THREADS), 0, s, a);
}

template <int MODE, int W>
bool launch_resident(const Args& a, unsigned grid, hipStream_t s) {
    size_t groups = (a.cols + W - 1) / W;
    if (groups <= 64 * 2) launch_cfg<MODE, 64, 2, W>(a, grid, s);
    else if (groups <= 64 * 8) launch_cfg<MODE, 64, 8, W>(a, grid, s);
    else if (groups <= 256 * 2) launch_cfg<MODE, 256, 2, W>(a, grid, s);
    else if (groups <= 256 * 8) launch_cfg<MODE, 256, 8, W>(a, grid, s);
    else if (groups <= 1024 * 2) launch_cfg<MODE, 1024, 2, W>(a, grid, s);
    else if (groups <= 1024 * 8) launch_cfg<MODE, 1024, 8, W>(a, grid, s);
    else return false;
    return true;
}

template <int MODE>
int run_rows(const char* name, Args a, float* loss_out, void* stream) {
    constexpr bool kLoss = (MODE == kCeOnehot || MODE == kCeIndex);
    if (kLoss && !loss_out) return fail(CTAMD_EINVAL, "%s: null output", name);
    hipStream_t s = as_stream(stream);
    if (a.rows == 0 || a.cols == 0) {
        if (kLoss) return ctamd_fill_f32(loss_out, 0.0f, 1, stream);
        return CTAMD_OK;
    }
    if (!a.x || (!a.t && MODE != kSoftmax)) return fail(CTAMD_EINVAL, "%s: null input", name);
    if (!kLoss && !a.out) return fail(CTAMD_EINVAL, "%s: null output", name);
    if ((MODE == kCeBwdOnehot || MODE == kCeBwdIndex) && !a.g1) return fail(CTAMD_EINVAL, "%s: null upstream gradient", name);
    if (a.rows > (size_t(1) << 62) / a.cols) return fail(CTAMD_ERANGE, "%s: rows*cols overflows", name);
    if (a.cols > size_t(0x7fffffff)) return fail(CTAMD_ERANGE, "%s: more than 2^31-1 columns", name);
    if (kLoss) {
        a.partials = reinterpret_cast<double*>(scratch());
        if (!a.partials) return CTAMD_EINVAL;
    }
    unsigned grid = a.rows < kMaxRowBlocks ? unsigned(a.rows) : kMaxRowBlocks;
    bool vec = (a.cols % 4 == 0) && aligned16(a.x) && (MODE == kSoftmax || MODE == kCeIndex || MODE == kCeBwdIndex || aligned16(a.t)) &&
               (kLoss || aligned16(a.out));
    bool done = vec ? launch_resident<MODE, 4>(a, grid, s) : launch_resident<MODE, 1>(a, grid, s);
    if (!done) hipLaunchKernelGGL((row_stream_kernel<MODE>), dim3(grid), dim3(1024), 0, s, a);
    int rc = launched(name);
    if (rc) return rc;
    if (kLoss) {
        hipLaunchKernelGGL(loss_stage2, dim3(1), dim3(256), 0, s, a.partials, grid, loss_out);
        rc = launched(name);
    }
    return rc;
}

// ---------------------------------------------------------------- column (dim 0) variants
// One thread per column, rows walked in order (adjacent threads touch adjacent addresses).
__global__ __launch_bounds__(256) void softmax_cols_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                           size_t rows, size_t cols) {
    __shared__ uint64_t s_exp2[32];
    stage_exp_table(s_exp2);
    size_t j = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (j >= cols) return;
    float m = x[j];
    for (size_t i = 1; i < rows; ++i) {
        float v = x[i * cols + j];
        if (v > m) m = v;
    }
    float s = 0.0f;
    for (size_t i = 0; i < rows; ++i) {
        float e = cta_expf_tab(x[i * cols + j] - m, s_exp2);
        y[i * cols + j] = e;
        s += e;
    }
    for (size_t i = 0; i < rows; ++i) y[i * cols + j] /= s;
}
__global__ __launch_bounds__(256) void softmax_bwd_cols_kernel(const float* __restrict__ y, const float* __restrict__ g,
                                                               float* __restrict__ dx, size_t rows, size_t cols) {
    size_t j = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (j >= cols) return;
    float d = 0.0f;
    for (size_t i = 0; i < rows; ++i) d = __fmaf_rn(g[i * cols + j], y[i * cols + j], d);
    for (size_t i = 0; i < rows; ++i) dx[i * cols + j] = y[i * cols + j] * (g[i * cols + j] - d);
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols, void* stream) {
    Args a{x, nullptr, nullptr, y, nullptr, nullptr, rows, cols};
    return run_rows<kSoftmax>(__func__, a, nullptr, stream);
}
int ctamd_cross_entropy_onehot_f32(const float* x, const float* t, float* out, size_t rows, size_t cols, void* stream) {
    Args a{x, t, nullptr, nullptr, nullptr, nullptr, rows, cols};
    return run_rows<kCeOnehot>(__func__, a, out, stream);
}
int ctamd_cross_entropy_index_f32(const float* x, const float* idx, float* out, int32_t* status, size_t rows,
                                  size_t cols, void* stream) {
    if (status) {   // cleared by a kernel, not a memset node, so that callers may capture this call
        hipLaunchKernelGGL(clear_i32, dim3(1), dim3(1), 0, as_stream(stream), status);
        int rc = launched(__func__);
        if (rc) return rc;
    }
    Args a{x, idx, nullptr, nullptr, nullptr, status, rows, cols};
    return run_rows<kCeIndex>(__func__, a, out, stream);
}
int ctamd_cross_entropy_backward_onehot_f32(const float* x, const float* t, const float* g1, float* dx, size_t rows,
                                            size_t cols, void* stream) {
    Args a{x, t, g1, dx, nullptr, nullptr, rows, cols};
    return run_rows<kCeBwdOnehot>(__func__, a, nullptr, stream);
}
int ctamd_cross_entropy_backward_index_f32(const float* x, const float* idx, const float* g1, float* dx, size_t rows,
                                           size_t cols, void* stream) {
    Args a{x, idx, g1, dx, nullptr, nullptr, rows, cols};
    return run_rows<kCeBwdIndex>(__func__, a, nullptr, stream);
}
int ctamd_softmax_backward_rows_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream) {
    Args a{y, g, nullptr, dx, nullptr, nullptr, rows, cols};
    return run_rows<kSoftmaxBwd>(__func__, a, nullptr, stream);
}

int ctamd_softmax_cols_f32(const float* x, float* y, size_t rows, size_t cols, void* stream) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!x || !y) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    hipLaunchKernelGGL(softmax_cols_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, as_stream(stream), x, y,
                       rows, cols);
    return launched(__func__);
}
int ctamd_softmax_backward_cols_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!y || !g || !dx) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    hipLaunchKernelGGL(softmax_bwd_cols_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, as_stream(stream), y,
                       g, dx, rows, cols);
    return launched(__func__);
}

}  // extern "C"
