// The reference's arms for tensors that are not fp32 (double, int32, int64, bool): zero() / ones(),
// Tensor::to(dtype) from fp32, tensor (+ * /) float, the in-place gradient accumulation, and the
// double softmax.  All but the softmax are HBM streams of 16-byte vectors; integer arithmetic wraps
// (computed unsigned) and fp32 -> integer conversion gives the x86 "integer indefinite" value for
// NaN and out-of-range inputs, which is what the reference's build computes.
#include <limits.h>

#include "common.h"
#include "devmath.h"

namespace ctamd {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;

// what a lane moves at once: 16 bytes (bool: four bytes, so that the fp32 source of a conversion
// is one 16-byte vector as well)
template <class T>
struct Vec {
    static constexpr int kLanes = sizeof(T) == 1 ? 4 : 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(sizeof(T) == 1 ? 4 : 16 / sizeof(T))));
};

// static_cast<int32_t / int64_t>(float) as cvttss2si computes it: truncation, 0x80..0 otherwise
__device__ __forceinline__ int32_t to_i32(float x) {
    return (x >= -2147483648.0f && x < 2147483648.0f) ? int32_t(x) : INT32_MIN;
}
__device__ __forceinline__ int64_t to_i64(float x) {
    return (x >= -9223372036854775808.0f && x < 9223372036854775808.0f) ? int64_t(x) : INT64_MIN;
}
inline int32_t host_to_i32(float x) { return (x >= -2147483648.0f && x < 2147483648.0f) ? int32_t(x) : INT32_MIN; }
inline int64_t host_to_i64(float x) {
    return (x >= -9223372036854775808.0f && x < 9223372036854775808.0f) ? int64_t(x) : INT64_MIN;
}

template <class T>
__device__ __forceinline__ T cast_one(float x);
template <>
__device__ __forceinline__ double cast_one<double>(float x) { return double(x); }
template <>
__device__ __forceinline__ int32_t cast_one<int32_t>(float x) { return to_i32(x); }
template <>
__device__ __forceinline__ int64_t cast_one<int64_t>(float x) { return to_i64(x); }
template <>
__device__ __forceinline__ uint8_t cast_one<uint8_t>(float x) { return x != 0.0f ? 1 : 0; }   // NaN is true

enum { kAdd = CTAMD_TS_ADD, kMul = CTAMD_TS_MUL, kDiv = CTAMD_TS_DIV };

template <int OP>
__device__ __forceinline__ double op_one(double x, double s) { return OP == kAdd ? x + s : OP == kMul ? x * s : x / s; }
template <int OP>
__device__ __forceinline__ int32_t op_one(int32_t x, int32_t s) {
    if (OP == kAdd) return int32_t(uint32_t(x) + uint32_t(s));
    if (OP == kMul) return int32_t(uint32_t(x) * uint32_t(s));
    return (s == -1) ? int32_t(0u - uint32_t(x)) : x / s;       // INT_MIN / -1 wraps instead of trapping
}
template <int OP>
__device__ __forceinline__ int64_t op_one(int64_t x, int64_t s) {
    if (OP == kAdd) return int64_t(uint64_t(x) + uint64_t(s));
    if (OP == kMul) return int64_t(uint64_t(x) * uint64_t(s));
    return (s == -1) ? int64_t(uint64_t(0) - uint64_t(x)) : x / s;
}

// out[i] = f(i-th vector); a thread owns kUnroll vectors one block-width apart, loaded (through
// `load`) before the first is used; the tail beyond the last whole vector goes element by element
// to the first threads of the grid.
template <class T, class LoadF, class ElemF>
__device__ __forceinline__ void stream_out(T* __restrict__ out, size_t n, LoadF load, ElemF elem) {
    typedef typename Vec<T>::type V;
    constexpr int L = Vec<T>::kLanes;
    const size_t nv = n / L;
    const size_t per_block = size_t(kThreads) * kUnroll;
    for (size_t base = size_t(blockIdx.x) * per_block; base < nv; base += size_t(gridDim.x) * per_block) {
        V r[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t i = base + size_t(u) * kThreads + threadIdx.x;
            if (i < nv) r[u] = load(i);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t i = base + size_t(u) * kThreads + threadIdx.x;
            if (i < nv) __builtin_nontemporal_store(r[u], reinterpret_cast<V*>(out) + i);
        }
    }
    const size_t t = size_t(blockIdx.x) * kThreads + threadIdx.x;
    if (t < n - nv * L) out[nv * L + t] = elem(nv * L + t);
}

template <class T>
__global__ __launch_bounds__(kThreads) void fill_typed_kernel(T* __restrict__ out, T v, size_t n) {
    typedef typename Vec<T>::type V;
    stream_out<T>(out, n, [&](size_t) { V r; for (int e = 0; e < Vec<T>::kLanes; ++e) r[e] = v; return r; },
                  [&](size_t) { return v; });
}

template <class T>
__global__ __launch_bounds__(kThreads) void cast_kernel(const float* __restrict__ in, T* __restrict__ out, size_t n) {
    typedef typename Vec<T>::type V;
    typedef float F __attribute__((ext_vector_type(Vec<T>::kLanes)));
    stream_out<T>(out, n,
                  [&](size_t i) {
                      F x = __builtin_nontemporal_load(reinterpret_cast<const F*>(in) + i);
                      V r;
#pragma unroll
                      for (int e = 0; e < Vec<T>::kLanes; ++e) r[e] = cast_one<T>(x[e]);
                      return r;
                  },
                  [&](size_t i) { return cast_one<T>(in[i]); });
}

template <class T, int OP>
__global__ __launch_bounds__(kThreads) void scalar_typed_kernel(const T* __restrict__ in, T* __restrict__ out, T s, size_t n) {
    typedef typename Vec<T>::type V;
    stream_out<T>(out, n,
                  [&](size_t i) {
                      V x = __builtin_nontemporal_load(reinterpret_cast<const V*>(in) + i);
                      V r;
#pragma unroll
                      for (int e = 0; e < Vec<T>::kLanes; ++e) r[e] = op_one<OP>(T(x[e]), s);
                      return r;
                  },
                  [&](size_t i) { return op_one<OP>(in[i], s); });
}

template <class T>
__global__ __launch_bounds__(kThreads) void accumulate_typed_kernel(T* __restrict__ acc, const T* __restrict__ val, size_t n) {
    typedef typename Vec<T>::type V;
    stream_out<T>(acc, n,
                  [&](size_t i) {
                      V a = __builtin_nontemporal_load(reinterpret_cast<const V*>(acc) + i);
                      V b = __builtin_nontemporal_load(reinterpret_cast<const V*>(val) + i);
                      V r;
#pragma unroll
                      for (int e = 0; e < Vec<T>::kLanes; ++e) r[e] = op_one<kAdd>(T(a[e]), T(b[e]));
                      return r;
                  },
                  [&](size_t i) { return op_one<kAdd>(acc[i], val[i]); });
}

// One block per kThreads * kUnroll vectors, no cap: a block that makes one trip and exits measured
// faster on these streams than fewer blocks striding over the tensor (the loop in stream_out only
// serves tensors beyond 2^31 - 1 blocks).
template <class T>
unsigned typed_grid(size_t n) {
    const size_t per_block = size_t(kThreads) * kUnroll;
    const size_t need = (n / Vec<T>::kLanes + per_block) / per_block;
    return unsigned(need < 0x7fffffffu ? need : 0x7fffffffu);
}

// ------------------------------------------------------------------------------ double softmax

// The exponential is glibc's exp bit for bit (cta_exp64); its 2 KiB table of 2^(k/128) sits in LDS.
__device__ __forceinline__ void stage_exp64_table(uint64_t* tab) {
    for (unsigned i = threadIdx.x; i < 256; i += blockDim.x) tab[i] = cta_exp64_tab[i];
    __syncthreads();
}

__device__ __forceinline__ double block_reduce(double v, bool is_max, double* s_part) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        double o = __shfl_xor(v, off, 64);
        v = is_max ? (o > v ? o : v) : v + o;
    }
    const int wave = threadIdx.x >> 6;
    __syncthreads();                    // s_part may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) s_part[wave] = v;
    __syncthreads();
    double r = s_part[0];
    for (int w = 1; w < int(blockDim.x >> 6); ++w) r = is_max ? (s_part[w] > r ? s_part[w] : r) : r + s_part[w];
    return r;
}

// One block per row (grid-stride over rows): maximum, sum of exp(x - max), y = exp(x - max) / sum.
// The row is read three times (the second and third time from the caches for rows up to a few
// MiB) and the exponential computed twice, instead of being stored as the reference does.
__global__ __launch_bounds__(256) void softmax_rows_f64_kernel(const double* __restrict__ x, double* __restrict__ y, size_t rows,
                                                               size_t cols) {
    __shared__ double s_part[4];
    __shared__ uint64_t s_tab[256];
    stage_exp64_table(s_tab);
    for (size_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const double* xr = x + row * cols;
        double* yr = y + row * cols;
        double m = -__builtin_huge_val();
        for (size_t j = threadIdx.x; j < cols; j += blockDim.x) m = xr[j] > m ? xr[j] : m;
        m = block_reduce(m, true, s_part);
        double sum = 0.0;
        for (size_t j = threadIdx.x; j < cols; j += blockDim.x) sum += cta_exp64(xr[j] - m, s_tab);
        sum = block_reduce(sum, false, s_part);
        for (size_t j = threadIdx.x; j < cols; j += blockDim.x) yr[j] = cta_exp64(xr[j] - m, s_tab) / sum;
    }
}

// The same with the row in registers: every element is read once, its exponential computed once
// and kept (as the reference keeps it: src/Tensor.cpp:1686-1696), then divided by the row's sum.
// PAIRS 128-bit words (two doubles) per thread, 256 threads: rows of up to 512 * PAIRS columns;
// cols even and both pointers 16-byte aligned.
typedef double v2d __attribute__((ext_vector_type(2)));
template <int PAIRS>
__global__ __launch_bounds__(256) void softmax_rows_f64_resident_kernel(const double* __restrict__ x, double* __restrict__ y, size_t rows,
                                                                        size_t cols) {
    __shared__ double s_part[4];
    __shared__ uint64_t s_tab[256];
    stage_exp64_table(s_tab);
    const size_t pairs = cols / 2;
    for (size_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const v2d* xr = reinterpret_cast<const v2d*>(x + row * cols);
        v2d* yr = reinterpret_cast<v2d*>(y + row * cols);
        v2d v[PAIRS];
        double m = -__builtin_huge_val();
#pragma unroll
        for (int k = 0; k < PAIRS; ++k) {
            const size_t j = size_t(k) * 256 + threadIdx.x;
            v[k] = v2d{-__builtin_huge_val(), -__builtin_huge_val()};
            if (j < pairs) v[k] = __builtin_nontemporal_load(xr + j);
        }
#pragma unroll
        for (int k = 0; k < PAIRS; ++k) {
            m = v[k][0] > m ? v[k][0] : m;
            m = v[k][1] > m ? v[k][1] : m;
        }
        m = block_reduce(m, true, s_part);
        double sum = 0.0;
#pragma unroll
        for (int k = 0; k < PAIRS; ++k) {
            const size_t j = size_t(k) * 256 + threadIdx.x;
            if (j < pairs) {
                v[k][0] = cta_exp64(v[k][0] - m, s_tab);
                v[k][1] = cta_exp64(v[k][1] - m, s_tab);
                sum += v[k][0];
                sum += v[k][1];
            }
        }
        sum = block_reduce(sum, false, s_part);
#pragma unroll
        for (int k = 0; k < PAIRS; ++k) {
            const size_t j = size_t(k) * 256 + threadIdx.x;
            if (j < pairs) __builtin_nontemporal_store(v2d{v[k][0] / sum, v[k][1] / sum}, yr + j);
        }
    }
}

// Column softmax in three launches over chunks of rows, the layout of the fp32 column kernels: a
// block owns a strip of 256 * W neighbouring columns of one chunk (a row of the strip is 4 KiB of
// contiguous memory with two columns per thread) and every thread walks the chunk's rows in order,
// four rows' loads in flight.  First launch: a running (maximum, sum of exp(x - maximum)) pair per
// thread with ONE exponential per element - of the element's distance below the maximum, or of
// the old maximum's distance below the element when the maximum moves - kept apart for the even
// and odd rows of the chunk (two short dependency chains instead of one) and left per (chunk,
// column) in `pairs`.  Second launch: the chunks' pairs of a column brought to the column maximum
// and added in chunk-group order.  Third launch: y = exp(x - max) / sum, the quotient as a product
// with the column's reciprocal and one correction step (e r + fma(-(e r), sum, e) r: the correctly
// rounded quotient but for results in the subnormal range, where it is within one of their units).
// Two exponentials and 24 bytes per element.  (One thread walking a whole column, the reference's
// order src/Tensor.cpp:1766-1781, took 11.9 ms on [8192 x 8192]; blocks of 32 columns x 8 row
// groups, which read 512 bytes of a row at a time, and a true division per element: 345 us.)
struct MaxSum {
    double m, s;
};
__device__ __forceinline__ MaxSum join(MaxSum a, MaxSum b, const uint64_t* tab) {       // a's rows come before b's
    const double m = b.m > a.m ? b.m : a.m;
    MaxSum r;
    r.m = m;
    r.s = (a.s == 0.0 ? 0.0 : a.s * cta_exp64(a.m - m, tab)) + (b.s == 0.0 ? 0.0 : b.s * cta_exp64(b.m - m, tab));
    return r;
}
constexpr int kColRows = 4;             // rows whose loads are in flight
// W columns per thread: 2 with 128-bit accesses (cols even, pointers 16-byte aligned), else 1.
template <int W>
__device__ __forceinline__ void load_cols(const double* __restrict__ p, double (&v)[W]) {
    if (W == 2) {
        const v2d t = *reinterpret_cast<const v2d*>(p);
        v[0] = t[0];
        v[W - 1] = t[1];
    } else {
        v[0] = p[0];
    }
}
template <int W>
__global__ __launch_bounds__(256) void softmax_cols_f64_scan_kernel(const double* __restrict__ x, MaxSum* __restrict__ pairs, size_t rows,
                                                                    size_t cols, size_t rows_per_chunk) {
    __shared__ uint64_t s_tab[256];
    stage_exp64_table(s_tab);
    const size_t j = (size_t(blockIdx.x) * 256 + threadIdx.x) * W;
    if (j >= cols) return;
    const size_t first = size_t(blockIdx.y) * rows_per_chunk;
    size_t last = first + rows_per_chunk;
    if (last > rows) last = rows;
    MaxSum t[2][W];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int w = 0; w < W; ++w) t[h][w] = MaxSum{-__builtin_huge_val(), 0.0};
    auto one_row = [&](int h, const double (&v)[W]) {
#pragma unroll
        for (int w = 0; w < W; ++w) {
            MaxSum& q = t[h][w];
            const bool up = v[w] > q.m;
            const double e = cta_exp64(up ? q.m - v[w] : v[w] - q.m, s_tab);      // q.m = -inf at the start: exp(-inf) = 0
            q.s = up ? q.s * e + 1.0 : q.s + e;
            q.m = up ? v[w] : q.m;
        }
    };
    const double* __restrict__ p = x + first * cols + j;
    size_t i = first;
    for (; i + kColRows <= last; i += kColRows, p += kColRows * cols) {
        double v[kColRows][W];
#pragma unroll
        for (int r = 0; r < kColRows; ++r) load_cols<W>(p + size_t(r) * cols, v[r]);
#pragma unroll
        for (int r = 0; r < kColRows; ++r) one_row(r & 1, v[r]);
    }
    for (; i < last; ++i, p += cols) {
        double v[W];
        load_cols<W>(p, v);
        if ((i - first) & 1) one_row(1, v);              // constant indices keep the accumulators in registers
        else one_row(0, v);
    }
#pragma unroll
    for (int w = 0; w < W; ++w) pairs[size_t(blockIdx.y) * cols + j + w] = join(t[0][w], t[1][w], s_tab);
}
// A block folds 16 columns; its 64 groups of 16 lanes take every 64th chunk, and the groups are
// combined through LDS in group order (every CU takes part: a CU alone draws little bandwidth).
constexpr int kFoldCols64 = 16, kFoldGroups64 = 64;
__global__ __launch_bounds__(kFoldCols64 * kFoldGroups64) void softmax_cols_f64_fold_kernel(const MaxSum* __restrict__ pairs,
                                                                                          MaxSum* __restrict__ totals, size_t cols,
                                                                                          unsigned chunks) {
    __shared__ uint64_t s_tab[256];
    __shared__ double s_m[kFoldGroups64][kFoldCols64], s_s[kFoldGroups64][kFoldCols64];
    stage_exp64_table(s_tab);
    const unsigned lane = threadIdx.x % kFoldCols64, group = threadIdx.x / kFoldCols64;
    const size_t c = size_t(blockIdx.x) * kFoldCols64 + lane;
    const bool live = c < cols;
    double m = -__builtin_huge_val();
    if (live)
        for (unsigned k = group; k < chunks; k += kFoldGroups64) {
            const double v = pairs[size_t(k) * cols + c].m;
            m = v > m ? v : m;
        }
    s_m[group][lane] = m;
    __syncthreads();
#pragma unroll 8
    for (int g = 0; g < kFoldGroups64; ++g) m = s_m[g][lane] > m ? s_m[g][lane] : m;
    double sum = 0.0;
    if (live)
        for (unsigned k = group; k < chunks; k += kFoldGroups64) {
            const MaxSum q = pairs[size_t(k) * cols + c];
            sum += q.s == 0.0 ? 0.0 : q.s * cta_exp64(q.m - m, s_tab);
        }
    s_s[group][lane] = sum;
    __syncthreads();
    if (group == 0 && live) {
        double total = 0.0;
#pragma unroll 8
        for (int g = 0; g < kFoldGroups64; ++g) total += s_s[g][lane];
        totals[c] = MaxSum{m, total};
    }
}
template <int W>
__global__ __launch_bounds__(256) void softmax_cols_f64_write_kernel(const double* __restrict__ x, const MaxSum* __restrict__ totals,
                                                                     double* __restrict__ y, size_t rows, size_t cols,
                                                                     size_t rows_per_chunk) {
    __shared__ uint64_t s_tab[256];
    stage_exp64_table(s_tab);
    const size_t j = (size_t(blockIdx.x) * 256 + threadIdx.x) * W;
    if (j >= cols) return;
    double m[W], sum[W], inv[W];
#pragma unroll
    for (int w = 0; w < W; ++w) {
        const MaxSum q = totals[j + w];
        m[w] = q.m;
        sum[w] = q.s;
        inv[w] = 1.0 / q.s;
    }
    const size_t first = size_t(blockIdx.y) * rows_per_chunk;
    size_t last = first + rows_per_chunk;
    if (last > rows) last = rows;
    auto one_row = [&](const double (&v)[W], double* __restrict__ dst) {
        double o[W];
#pragma unroll
        for (int w = 0; w < W; ++w) {
            const double e = cta_exp64(v[w] - m[w], s_tab);
            const double q0 = e * inv[w];
            o[w] = __builtin_fma(__builtin_fma(-q0, sum[w], e), inv[w], q0);
        }
        if (W == 2) __builtin_nontemporal_store(v2d{o[0], o[W - 1]}, reinterpret_cast<v2d*>(dst));
        else dst[0] = o[0];
    };
    const double* __restrict__ p = x + first * cols + j;
    double* __restrict__ d = y + first * cols + j;
    size_t i = first;
    for (; i + kColRows <= last; i += kColRows, p += kColRows * cols, d += kColRows * cols) {
        double v[kColRows][W];
#pragma unroll
        for (int r = 0; r < kColRows; ++r) load_cols<W>(p + size_t(r) * cols, v[r]);
#pragma unroll
        for (int r = 0; r < kColRows; ++r) one_row(v[r], d + size_t(r) * cols);
    }
    for (; i < last; ++i, p += cols, d += cols) {
        double v[W];
        load_cols<W>(p, v);
        one_row(v, d);
    }
}

size_t dtype_bytes(int dtype) {
    switch (dtype) {
        case CTAMD_DT_F32: case CTAMD_DT_I32: return 4;
        case CTAMD_DT_F64: case CTAMD_DT_I64: return 8;
        case CTAMD_DT_BOOL: return 1;
    }
    return 0;
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_fill_typed(void* out, int dtype, double value, size_t n, void* stream) {
    const size_t width = dtype_bytes(dtype);
    if (!width) return fail(CTAMD_EINVAL, "%s: bad dtype %d", __func__, dtype);
    if (n == 0) return CTAMD_OK;
    if (!out) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    if (!aligned16(out)) return fail(CTAMD_EINVAL, "%s: the tensor must start on a 16-byte boundary", __func__);
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case CTAMD_DT_F32:
            hipLaunchKernelGGL(fill_typed_kernel<float>, dim3(typed_grid<float>(n)), dim3(kThreads), 0, s, static_cast<float*>(out), float(value), n);
            break;
        case CTAMD_DT_F64:
            hipLaunchKernelGGL(fill_typed_kernel<double>, dim3(typed_grid<double>(n)), dim3(kThreads), 0, s, static_cast<double*>(out), value, n);
            break;
        case CTAMD_DT_I32:
            hipLaunchKernelGGL(fill_typed_kernel<int32_t>, dim3(typed_grid<int32_t>(n)), dim3(kThreads), 0, s, static_cast<int32_t*>(out),
                               int32_t(value), n);
            break;
        case CTAMD_DT_I64:
            hipLaunchKernelGGL(fill_typed_kernel<int64_t>, dim3(typed_grid<int64_t>(n)), dim3(kThreads), 0, s, static_cast<int64_t*>(out),
                               int64_t(value), n);
            break;
        default: {      // whole 32-bit words of four equal bytes, then the last 0..3 bytes
            const uint8_t b = value != 0.0 ? 1 : 0;
            const size_t words = n / 4;
            if (words)
                hipLaunchKernelGGL(fill_typed_kernel<int32_t>, dim3(typed_grid<int32_t>(words)), dim3(kThreads), 0, s, static_cast<int32_t*>(out),
                                   int32_t(b * 0x01010101u), words);
            if (n % 4)
                hipLaunchKernelGGL(fill_typed_kernel<uint8_t>, dim3(1), dim3(kThreads), 0, s, static_cast<uint8_t*>(out) + words * 4, b, n % 4);
        }
    }
    account(double(n) * double(width), 0.0);
    return launched(__func__);
}

int ctamd_cast_from_f32(const float* in, void* out, int dtype, size_t n, void* stream) {
    const size_t width = dtype_bytes(dtype);
    if (!width || dtype == CTAMD_DT_F32) return fail(CTAMD_EINVAL, "%s: bad target dtype %d", __func__, dtype);
    if (n == 0) return CTAMD_OK;
    if (!in || !out) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    if (!aligned16(out) || !aligned16(in)) return fail(CTAMD_EINVAL, "%s: tensors must start on 16-byte boundaries", __func__);
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case CTAMD_DT_F64:
            hipLaunchKernelGGL(cast_kernel<double>, dim3(typed_grid<double>(n)), dim3(kThreads), 0, s, in, static_cast<double*>(out), n);
            break;
        case CTAMD_DT_I32:
            hipLaunchKernelGGL(cast_kernel<int32_t>, dim3(typed_grid<int32_t>(n)), dim3(kThreads), 0, s, in, static_cast<int32_t*>(out), n);
            break;
        case CTAMD_DT_I64:
            hipLaunchKernelGGL(cast_kernel<int64_t>, dim3(typed_grid<int64_t>(n)), dim3(kThreads), 0, s, in, static_cast<int64_t*>(out), n);
            break;
        default:
            hipLaunchKernelGGL(cast_kernel<uint8_t>, dim3(typed_grid<uint8_t>(n)), dim3(kThreads), 0, s, in, static_cast<uint8_t*>(out), n);
    }
    account(double(n) * double(4 + width), 0.0);
    return launched(__func__);
}

int ctamd_scalar_op_typed(const void* in, void* out, int dtype, int op, float scalar, size_t n, void* stream) {
    if (dtype != CTAMD_DT_F64 && dtype != CTAMD_DT_I32 && dtype != CTAMD_DT_I64)
        return fail(CTAMD_EINVAL, "%s: dtype %d has no scalar arithmetic", __func__, dtype);
    if (op != kAdd && op != kMul && op != kDiv) return fail(CTAMD_EINVAL, "%s: bad op %d", __func__, op);
    const int64_t si = dtype == CTAMD_DT_I32 ? int64_t(host_to_i32(scalar)) : host_to_i64(scalar);
    if (op == kDiv && dtype != CTAMD_DT_F64 && si == 0)
        return fail(CTAMD_EINVAL, "%s: the scalar converts to the integer 0 (the reference's process stops on this division)", __func__);
    if (n == 0) return CTAMD_OK;
    if (!in || !out) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    if (!aligned16(out) || !aligned16(in)) return fail(CTAMD_EINVAL, "%s: tensors must start on 16-byte boundaries", __func__);
    hipStream_t s = as_stream(stream);
#define CTAMD_TYPED_LAUNCH(T, OP, SV) \
    hipLaunchKernelGGL((scalar_typed_kernel<T, OP>), dim3(typed_grid<T>(n)), dim3(kThreads), 0, s, static_cast<const T*>(in), static_cast<T*>(out), T(SV), n)
#define CTAMD_TYPED_OPS(T, SV)                              \
    do {                                                    \
        if (op == kAdd) CTAMD_TYPED_LAUNCH(T, kAdd, SV);    \
        else if (op == kMul) CTAMD_TYPED_LAUNCH(T, kMul, SV); \
        else CTAMD_TYPED_LAUNCH(T, kDiv, SV);               \
    } while (0)
    if (dtype == CTAMD_DT_F64) CTAMD_TYPED_OPS(double, double(scalar));
    else if (dtype == CTAMD_DT_I32) CTAMD_TYPED_OPS(int32_t, si);
    else CTAMD_TYPED_OPS(int64_t, si);
#undef CTAMD_TYPED_OPS
#undef CTAMD_TYPED_LAUNCH
    account(double(n) * 2.0 * double(dtype_bytes(dtype)), 0.0);
    return launched(__func__);
}

int ctamd_accumulate_typed(void* acc, const void* val, int dtype, size_t n, void* stream) {
    if (dtype != CTAMD_DT_F64 && dtype != CTAMD_DT_I32 && dtype != CTAMD_DT_I64)
        return fail(CTAMD_EINVAL, "%s: dtype %d is not accumulated", __func__, dtype);
    if (n == 0) return CTAMD_OK;
    if (!acc || !val) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    if (!aligned16(acc) || !aligned16(val)) return fail(CTAMD_EINVAL, "%s: tensors must start on 16-byte boundaries", __func__);
    hipStream_t s = as_stream(stream);
    if (dtype == CTAMD_DT_F64)
        hipLaunchKernelGGL(accumulate_typed_kernel<double>, dim3(typed_grid<double>(n)), dim3(kThreads), 0, s, static_cast<double*>(acc),
                           static_cast<const double*>(val), n);
    else if (dtype == CTAMD_DT_I32)
        hipLaunchKernelGGL(accumulate_typed_kernel<int32_t>, dim3(typed_grid<int32_t>(n)), dim3(kThreads), 0, s, static_cast<int32_t*>(acc),
                           static_cast<const int32_t*>(val), n);
    else
        hipLaunchKernelGGL(accumulate_typed_kernel<int64_t>, dim3(typed_grid<int64_t>(n)), dim3(kThreads), 0, s, static_cast<int64_t*>(acc),
                           static_cast<const int64_t*>(val), n);
    account(double(n) * 3.0 * double(dtype_bytes(dtype)), 0.0);
    return launched(__func__);
}

int ctamd_softmax_f64(const double* x, double* y, size_t rows, size_t cols, int dim, void* stream) {
    if (dim != 0 && dim != 1) return fail(CTAMD_EINVAL, "%s: dim must be 0 or 1", __func__);
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!x || !y) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    hipStream_t s = as_stream(stream);
    if (dim == 1) {
        const unsigned blocks = stream_grid(rows, 1, 8);
        const bool pairs_ok = cols % 2 == 0 && aligned16(x) && aligned16(y);
        if (pairs_ok && cols > 64 && cols <= 512) hipLaunchKernelGGL(softmax_rows_f64_resident_kernel<1>, dim3(blocks), dim3(256), 0, s, x, y, rows, cols);
        else if (pairs_ok && cols > 64 && cols <= 1024) hipLaunchKernelGGL(softmax_rows_f64_resident_kernel<2>, dim3(blocks), dim3(256), 0, s, x, y, rows, cols);
        else if (pairs_ok && cols > 64 && cols <= 2048) hipLaunchKernelGGL(softmax_rows_f64_resident_kernel<4>, dim3(blocks), dim3(256), 0, s, x, y, rows, cols);
        else if (pairs_ok && cols > 64 && cols <= 4096) hipLaunchKernelGGL(softmax_rows_f64_resident_kernel<8>, dim3(blocks), dim3(256), 0, s, x, y, rows, cols);
        else if (pairs_ok && cols > 64 && cols <= 8192) hipLaunchKernelGGL(softmax_rows_f64_resident_kernel<16>, dim3(blocks), dim3(256), 0, s, x, y, rows, cols);
        else hipLaunchKernelGGL(softmax_rows_f64_kernel, dim3(blocks), dim3(cols <= 64 ? 64 : 256), 0, s, x, y, rows, cols);
    } else {
        const bool wide = cols % 2 == 0 && aligned16(x) && aligned16(y);
        const size_t per_block = size_t(256) * (wide ? 2 : 1);
        // (Column panels of 64 - 128 MiB, scanned and written in turn so that the writing launch would find
        // its panel in the memory-side cache, were measured: 445 us against 345 us for the whole matrix
        // at once on [8192 x 8192] - a panel's launches are too small to fill the chip.)
        const size_t strips = (cols + per_block - 1) / per_block;
        if (strips > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: too many columns", __func__);
        ScratchUse use(stream);
        MaxSum* pairs = reinterpret_cast<MaxSum*>(use.ptr());
        if (!pairs) return CTAMD_EINVAL;
        // chunks of at least 32 rows, at most 256 of them (half as many ran the two sweeps 15% slower: they
        // are bound by the exponential's arithmetic and want the blocks), as many as the scratch holds
        // pairs for beside the columns' totals
        const size_t slots = kScratchFloats * sizeof(float) / sizeof(MaxSum);
        if (cols > slots / 2) return fail(CTAMD_ERANGE, "%s: more than %zu columns", __func__, slots / 2);
        size_t chunks = (rows + 31) / 32;
        if (chunks > 256) chunks = 256;
        const size_t room = (slots - cols) / cols;
        if (chunks > room) chunks = room;
        const size_t rows_per_chunk = (rows + chunks - 1) / chunks;
        chunks = (rows + rows_per_chunk - 1) / rows_per_chunk;
        MaxSum* totals = pairs + chunks * cols;
        const dim3 grid{unsigned(strips), unsigned(chunks), 1u};
        const dim3 fold_grid{unsigned((cols + kFoldCols64 - 1) / kFoldCols64), 1u, 1u};
        if (wide) hipLaunchKernelGGL(softmax_cols_f64_scan_kernel<2>, grid, dim3(256), 0, s, x, pairs, rows, cols, rows_per_chunk);
        else hipLaunchKernelGGL(softmax_cols_f64_scan_kernel<1>, grid, dim3(256), 0, s, x, pairs, rows, cols, rows_per_chunk);
        hipLaunchKernelGGL(softmax_cols_f64_fold_kernel, fold_grid, dim3(kFoldCols64 * kFoldGroups64), 0, s, pairs, totals, cols, unsigned(chunks));
        if (wide) hipLaunchKernelGGL(softmax_cols_f64_write_kernel<2>, grid, dim3(256), 0, s, x, totals, y, rows, cols, rows_per_chunk);
        else hipLaunchKernelGGL(softmax_cols_f64_write_kernel<1>, grid, dim3(256), 0, s, x, totals, y, rows, cols, rows_per_chunk);
    }
    account(double(rows) * double(cols) * 16.0, 0.0);
    return launched(__func__);
}

}  // extern "C"
