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

// Column softmax in two launches over chunks of rows.  A block owns 32 neighbouring columns of one
// chunk; its 8 groups of 32 lanes take every 8th row of the chunk (a group reads 256 contiguous
// bytes per row).  First launch: a running (maximum, sum of exp(x - maximum)) pair per thread with
// ONE exponential per element - of the element's distance below the maximum, or of the old
// maximum's distance below the element when the maximum moves - combined over the groups in group
// order and left per (chunk, column) in `pairs`.  Second launch: every block brings the chunks' pairs
// of its columns to the column maximum in chunk order (a few exponentials per column), then writes
// y = exp(x - max) / sum.  Two exponentials and 24 bytes per element, against three sweeps of the
// whole matrix by 256 blocks before.  (One thread walking a whole column, the reference's order
// src/Tensor.cpp:1766-1781, took 11.9 ms on [8192 x 8192].)
constexpr int kLanesPerRow = 32, kRowGroups = 8;
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
// W columns per lane: 2 with 128-bit accesses (cols even, pointers 16-byte aligned), else 1.
template <int W>
__global__ __launch_bounds__(256) void softmax_cols_f64_scan_kernel(const double* __restrict__ x, MaxSum* __restrict__ pairs, size_t rows,
                                                                    size_t cols, size_t rows_per_chunk, size_t col0, size_t col_end) {
    __shared__ MaxSum s_red[kRowGroups][kLanesPerRow * W];
    __shared__ uint64_t s_tab[256];
    stage_exp64_table(s_tab);
    const unsigned lane = threadIdx.x % kLanesPerRow, group = threadIdx.x / kLanesPerRow;
    const size_t j = col0 + (size_t(blockIdx.x) * kLanesPerRow + lane) * W;
    const size_t first = size_t(blockIdx.y) * rows_per_chunk;
    size_t last = first + rows_per_chunk;
    if (last > rows) last = rows;
    MaxSum t[W];
#pragma unroll
    for (int w = 0; w < W; ++w) t[w] = MaxSum{-__builtin_huge_val(), 0.0};
    if (j < col_end) {
#pragma unroll 4
        for (size_t i = first + group; i < last; i += kRowGroups) {
            double v[W];
            if (W == 2) {
                const v2d p = *reinterpret_cast<const v2d*>(x + i * cols + j);
                v[0] = p[0];
                v[W - 1] = p[1];
            } else {
                v[0] = x[i * cols + j];
            }
#pragma unroll
            for (int w = 0; w < W; ++w) {
                const bool up = v[w] > t[w].m;
                const double e = cta_exp64(up ? t[w].m - v[w] : v[w] - t[w].m, s_tab);   // t.m = -inf at the start: exp(-inf) = 0
                t[w].s = up ? t[w].s * e + 1.0 : t[w].s + e;
                t[w].m = up ? v[w] : t[w].m;
            }
        }
    }
#pragma unroll
    for (int w = 0; w < W; ++w) s_red[group][lane * W + w] = t[w];
    __syncthreads();
    if (group == 0 && j < col_end) {
#pragma unroll
        for (int w = 0; w < W; ++w) {
            MaxSum r = s_red[0][lane * W + w];
#pragma unroll
            for (int g = 1; g < kRowGroups; ++g) r = join(r, s_red[g][lane * W + w], s_tab);
            pairs[size_t(blockIdx.y) * cols + j + w] = r;
        }
    }
}
template <int W>
__global__ __launch_bounds__(256) void softmax_cols_f64_write_kernel(const double* __restrict__ x, const MaxSum* __restrict__ pairs,
                                                                     double* __restrict__ y, size_t rows, size_t cols,
                                                                     size_t rows_per_chunk, unsigned chunks, size_t col0, size_t col_end) {
    __shared__ MaxSum s_total[kLanesPerRow * W];
    __shared__ uint64_t s_tab[256];
    stage_exp64_table(s_tab);
    const unsigned lane = threadIdx.x % kLanesPerRow, group = threadIdx.x / kLanesPerRow;
    const size_t j = col0 + (size_t(blockIdx.x) * kLanesPerRow + lane) * W;
    // The chunks' pairs of this block's columns, brought to the column maximum: first the maximum
    // over the chunks (no exponential), then the sums scaled to it - independent exponentials, added
    // in chunk order.  The block's 256 threads share the work: thread t takes column t % (32 W) and
    // every (256 / (32 W))-th chunk; the parts are added in part order.
    {
        constexpr int kCols = kLanesPerRow * W, kParts = 256 / kCols;
        __shared__ double s_m[kParts][kCols], s_s[kParts][kCols];
        const unsigned c_in = threadIdx.x % kCols, part = threadIdx.x / kCols;
        const size_t col = col0 + size_t(blockIdx.x) * kCols + c_in;
        double m = -__builtin_huge_val();
        if (col < col_end)
            for (unsigned c = part; c < chunks; c += kParts) {
                const double v = pairs[size_t(c) * cols + col].m;
                m = v > m ? v : m;
            }
        s_m[part][c_in] = m;
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kParts; ++q) m = s_m[q][c_in] > m ? s_m[q][c_in] : m;
        double sum = 0.0;
        if (col < col_end)
            for (unsigned c = part; c < chunks; c += kParts) {
                const MaxSum p = pairs[size_t(c) * cols + col];
                sum += p.s == 0.0 ? 0.0 : p.s * cta_exp64(p.m - m, s_tab);
            }
        s_s[part][c_in] = sum;
        __syncthreads();
        if (part == 0) {
            double total = 0.0;
#pragma unroll
            for (int q = 0; q < kParts; ++q) total += s_s[q][c_in];
            s_total[c_in] = MaxSum{m, total};
        }
    }
    __syncthreads();
    if (j >= col_end) return;
    MaxSum total[W];
#pragma unroll
    for (int w = 0; w < W; ++w) total[w] = s_total[lane * W + w];
    const size_t first = size_t(blockIdx.y) * rows_per_chunk;
    size_t last = first + rows_per_chunk;
    if (last > rows) last = rows;
#pragma unroll 4
    for (size_t i = first + group; i < last; i += kRowGroups) {
        if (W == 2) {
            const v2d p = *reinterpret_cast<const v2d*>(x + i * cols + j);
            const v2d q{cta_exp64(p[0] - total[0].m, s_tab) / total[0].s, cta_exp64(p[1] - total[W - 1].m, s_tab) / total[W - 1].s};
            __builtin_nontemporal_store(q, reinterpret_cast<v2d*>(y + i * cols + j));
        } else {
            y[i * cols + j] = cta_exp64(x[i * cols + j] - total[0].m, s_tab) / total[0].s;
        }
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
        const size_t per_block = size_t(kLanesPerRow) * (wide ? 2 : 1);
        // (Column panels of 64 - 128 MiB, scanned and written in turn so that the writing launch would find
        // its panel in the memory-side cache, were measured: 445 us against 345 us for the whole matrix
        // at once on [8192 x 8192] - a panel's launches are too small to fill the chip.)
        const size_t panel_cols = cols;
        const size_t cus = compute_units() > 0 ? size_t(compute_units()) : 256;
        MaxSum* pairs = reinterpret_cast<MaxSum*>(scratch(stream));
        if (!pairs) return CTAMD_EINVAL;
        for (size_t col0 = 0; col0 < cols; col0 += panel_cols) {
            const size_t col_end = col0 + panel_cols < cols ? col0 + panel_cols : cols;
            const size_t strips = (col_end - col0 + per_block - 1) / per_block;
            if (strips > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: too many columns", __func__);
            // chunks of rows so that the grid fills the chip (about eight blocks per CU), of at least 64
            // rows each, as many as the scratch holds pairs for
            size_t chunks = (8 * cus + strips - 1) / strips;
            if (chunks > (rows + 63) / 64) chunks = (rows + 63) / 64;
            const size_t room = kScratchFloats * sizeof(float) / sizeof(MaxSum) / cols;
            if (chunks > room) chunks = room;
            if (chunks > 65535) chunks = 65535;
            if (chunks < 1) return fail(CTAMD_ERANGE, "%s: more than %zu columns", __func__, kScratchFloats * sizeof(float) / sizeof(MaxSum));
            const size_t rows_per_chunk = (rows + chunks - 1) / chunks;
            chunks = (rows + rows_per_chunk - 1) / rows_per_chunk;
            const dim3 grid{unsigned(strips), unsigned(chunks), 1u};
            if (wide) {
                hipLaunchKernelGGL(softmax_cols_f64_scan_kernel<2>, grid, dim3(256), 0, s, x, pairs, rows, cols, rows_per_chunk, col0, col_end);
                hipLaunchKernelGGL(softmax_cols_f64_write_kernel<2>, grid, dim3(256), 0, s, x, pairs, y, rows, cols, rows_per_chunk, unsigned(chunks), col0, col_end);
            } else {
                hipLaunchKernelGGL(softmax_cols_f64_scan_kernel<1>, grid, dim3(256), 0, s, x, pairs, rows, cols, rows_per_chunk, col0, col_end);
                hipLaunchKernelGGL(softmax_cols_f64_write_kernel<1>, grid, dim3(256), 0, s, x, pairs, y, rows, cols, rows_per_chunk, unsigned(chunks), col0, col_end);
            }
        }
    }
    account(double(rows) * double(cols) * 16.0, 0.0);
    return launched(__func__);
}

}  // extern "C"
