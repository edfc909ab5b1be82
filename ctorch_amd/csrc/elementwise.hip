// Elementwise kernels: binary / broadcast / scalar / unary forward ops and the elementwise
// gradient arithmetic of the tape.  All of them are HBM-bound streams: one generic kernel moves
// 128-bit vectors (four in flight per thread and operand) and applies a per-element functor; the
// functors restate the reference's fp32 operation order exactly.  This file must be compiled with
// -ffp-contract=off: a fused multiply-add would change the bits.
#include "common.h"
#include "devmath.h"
#include "functors.h"

namespace ctamd {
namespace {

// -------------------------------------------------------------------------------- kernels

// A functor may turn itself into a cheaper one once per thread before the element loop
// (DevScalarF<DivF> reads its divisor and becomes DivByRcpF).
template <class F>
__device__ __forceinline__ F bind(const F& f) { return f; }
__device__ __forceinline__ DivByRcpF bind(const DevScalarF<DivF>& f) { return DivByRcpF{1.0 / double(*f.s)}; }

template <class F, class = void>
struct HasRare { static constexpr bool value = false; };
template <class F>
struct HasRare<F, decltype(void(F::kRare))> { static constexpr bool value = F::kRare; };

template <class F, class = void>
struct HasLogTable { static constexpr bool value = false; };
template <class F>
struct HasLogTable<F, decltype(void(F::kLogTable))> { static constexpr bool value = F::kLogTable; };

// One element: the functor's fast path, repaired through slow() when the functor flags the input.
template <class F, int NI>
__device__ __forceinline__ float apply1(const F& f, const float* x, const Tables& tabs) {
    if constexpr (HasRare<F>::value) {
        float o = f(x, tabs);
        if (__builtin_expect(f.rare(x), 0)) o = f.slow(x, tabs);
        return o;
    } else {
        return f(x, tabs);
    }
}

// 128-bit accesses with the non-temporal hint: these streams touch every byte once, and keeping
// them out of the caches' replacement order measured fastest on MI355X (6.2 TB/s for a + b at
// 256 MiB per operand, against 5.5 TB/s with plain accesses and 4.7 TB/s for a grid-stride loop
// whose four accesses per thread lie far apart).
// Small tensors (a chain of ops on a few MiB) keep plain accesses so that the next kernel finds
// its operands in L2 / Infinity Cache.  NT, chosen by the launcher from the bytes touched: 0 plain
// accesses, 1 hinted loads and a plain store (the result is small enough to be kept in the
// memory-side cache for its reader: result_streams()), 2 the hint on both sides.
template <int NT>
__device__ __forceinline__ v4f ld_stream(const float* p, size_t i4) {
    if (NT >= 1) return __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p) + i4);
    return reinterpret_cast<const v4f*>(p)[i4];
}
template <int NT>
__device__ __forceinline__ void st_stream(float* p, size_t i4, v4f v) {
    if (NT == 2) __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(p) + i4);
    else reinterpret_cast<v4f*>(p)[i4] = v;
}
// operands + result above this many bytes cannot stay cache resident (256 MiB Infinity Cache)
constexpr size_t kStreamBytes = size_t(64) << 20;
inline int hint_level(size_t all_bytes, size_t result_bytes) {
    return all_bytes >= kStreamBytes ? (result_streams(result_bytes) ? 2 : 1) : 0;
}

// The work of one thread of a vector block: its kUnroll vectors per operand, all loaded before the
// first use.  CHECK guards each vector against the end of the tensor (last block only).
template <class F, int NT, bool CHECK>
__device__ __forceinline__ void map_block(const Ptrs<F::kIn>& in, float* __restrict__ out, size_t n4, size_t base,
                                          const F& f, const Tables& tabs) {
    constexpr int NI = F::kIn;
    v4f v[NI > 0 ? NI : 1][kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + size_t(u) * kThreads;
        if (!CHECK || i < n4) {
#pragma unroll
            for (int k = 0; k < NI; ++k) v[k][u] = ld_stream<NT>(in.p[k], i);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + size_t(u) * kThreads;
        if (!CHECK || i < n4) {
            v4f o;
            bool rare = false;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x[NI > 0 ? NI : 1];
#pragma unroll
                for (int k = 0; k < NI; ++k) x[k] = v[k][u][e];
                o[e] = f(x, tabs);
                if constexpr (HasRare<F>::value) rare = rare || f.rare(x);
            }
            if constexpr (HasRare<F>::value) {
                if (__builtin_expect(rare, 0)) {
                    for (int e = 0; e < 4; ++e) {
                        float x[NI > 0 ? NI : 1];
                        for (int k = 0; k < NI; ++k) x[k] = v[k][u][e];
                        if (f.rare(x)) o[e] = f.slow(x, tabs);
                    }
                }
            }
            st_stream<NT>(out, i, o);
        }
    }
}

// VEC = true: all pointers 16-byte aligned.  Block b owns the kThreads*kUnroll consecutive
// vectors starting at b*kThreads*kUnroll (no loop: the grid covers the tensor), thread t takes
// vectors t, t+256, t+512, t+768 of that run, all loads issued before the first use.  The last
// n % 4 elements are handled by block 0.  VEC = false: scalar grid-stride (unaligned views).
template <class F, bool VEC, int NT>
__global__ __launch_bounds__(kThreads) void map_kernel(Ptrs<F::kIn> in, float* __restrict__ out, size_t n, F f_in) {
    __shared__ uint64_t s_exp2[F::kTables ? 32 : 1];
    __shared__ uint32_t s_pio4[F::kTables ? 24 : 1];
    __shared__ double s_log[HasLogTable<F>::value ? 32 : 1];
    if (F::kTables) stage_tables(s_exp2, s_pio4);
    if (HasLogTable<F>::value) stage_log_table(s_log);
    const Tables tabs{s_exp2, s_pio4, s_log};
    constexpr int NI = F::kIn;
    const auto f = bind(f_in);
    using B = decltype(bind(f_in));
    if (VEC) {
        const size_t n4 = n >> 2;
        const size_t block_base = size_t(blockIdx.x) * (kThreads * kUnroll);
        if (block_base + size_t(kThreads) * kUnroll <= n4)
            map_block<B, NT, false>(in, out, n4, block_base + threadIdx.x, f, tabs);   // interior block: no bounds checks
        else
            map_block<B, NT, true>(in, out, n4, block_base + threadIdx.x, f, tabs);
        if (blockIdx.x == 0) {
            size_t i = (n4 << 2) + threadIdx.x;
            if (i < n) {
                float x[NI > 0 ? NI : 1];
#pragma unroll
                for (int k = 0; k < NI; ++k) x[k] = in.p[k][i];
                out[i] = apply1<B, NI>(f, x, tabs);
            }
        }
    } else {
        const size_t tid = size_t(blockIdx.x) * kThreads + threadIdx.x;
        const size_t stride = size_t(gridDim.x) * kThreads;
        for (size_t i = tid; i < n; i += stride) {
            float x[NI > 0 ? NI : 1];
#pragma unroll
            for (int k = 0; k < NI; ++k) x[k] = in.p[k][i];
            out[i] = apply1<B, NI>(f, x, tabs);
        }
    }
}

template <class F>
int launch_map(const char* name, Ptrs<F::kIn> in, float* out, size_t n, F f, void* stream) {
    if (n == 0) return CTAMD_OK;
    if (!out) return fail(CTAMD_EINVAL, "%s: null output", name);
    bool vec = aligned16(out);
    for (int k = 0; k < F::kIn; ++k) {
        if (!in.p[k]) return fail(CTAMD_EINVAL, "%s: null input %d", name, k);
        vec = vec && aligned16(in.p[k]);
    }
    if (vec) {
        size_t blocks = (n / 4 + size_t(kThreads) * kUnroll - 1) / (size_t(kThreads) * kUnroll);
        if (blocks < 1) blocks = 1;
        if (blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: more than 2^43 elements", name);
        const int hint = hint_level(n * sizeof(float) * (F::kIn + 1), n * sizeof(float));
        if (hint == 2)
            hipLaunchKernelGGL((map_kernel<F, true, 2>), dim3(unsigned(blocks)), dim3(kThreads), 0, as_stream(stream), in, out, n, f);
        else if (hint == 1)
            hipLaunchKernelGGL((map_kernel<F, true, 1>), dim3(unsigned(blocks)), dim3(kThreads), 0, as_stream(stream), in, out, n, f);
        else
            hipLaunchKernelGGL((map_kernel<F, true, 0>), dim3(unsigned(blocks)), dim3(kThreads), 0, as_stream(stream), in, out, n, f);
    } else {
        unsigned grid = stream_grid(n, size_t(kThreads) * kUnroll);
        hipLaunchKernelGGL((map_kernel<F, false, 0>), dim3(grid), dim3(kThreads), 0, as_stream(stream), in, out, n, f);
    }
    account(double(F::kIn + 1) * 4.0 * double(n), 0.0);
    return launched(name);
}

// r[i,j] = a[i,j] (op) b[j].  VEC: cols % 4 == 0 and aligned pointers - every 128-bit vector of a
// meets one aligned vector of b (served from cache: b is cols*4 bytes, read rows times).
// r[i, j] = Op(a[i, j], b[j]) or, for an Op with kIn == 3, Op(a[i, j], b[j], g[i, j]).
template <class Op, bool VEC, class Index, int NT>
__global__ __launch_bounds__(kThreads) void rowbcast_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                            const float* __restrict__ g, float* __restrict__ r,
                                                            size_t total, Index cols) {
    const Tables tabs{nullptr, nullptr, nullptr};
    constexpr bool kThird = (Op::kIn == 3);
    if (VEC) {
        const size_t n4 = total >> 2;
        const Index cols4 = cols >> 2;
        const size_t base = size_t(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
        v4f va[kUnroll], vb[kUnroll], vg[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            size_t i = base + size_t(u) * kThreads;
            if (i < n4) {
                va[u] = ld_stream<NT>(a, i);
                if (kThird) vg[u] = ld_stream<NT>(g, i);
                vb[u] = reinterpret_cast<const v4f*>(b)[Index(i) % cols4];   // re-used: keep cached
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            size_t i = base + size_t(u) * kThreads;
            if (i < n4) {
                v4f o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x[3] = {va[u][e], vb[u][e], kThird ? vg[u][e] : 0.0f};
                    o[e] = Op()(x, tabs);
                }
                st_stream<NT>(r, i, o);
            }
        }
    } else {
        const size_t tid = size_t(blockIdx.x) * kThreads + threadIdx.x;
        const size_t stride = size_t(gridDim.x) * kThreads;
        for (size_t i = tid; i < total; i += stride) {
            float x[3] = {a[i], b[Index(i) % cols], kThird ? g[i] : 0.0f};
            r[i] = Op()(x, tabs);
        }
    }
}

template <class Op>
int launch_rowbcast(const char* name, const float* a, const float* b, float* r, size_t rows, size_t cols,
                    void* stream, const float* g = nullptr) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!a || !b || !r || (Op::kIn == 3 && !g)) return fail(CTAMD_EINVAL, "%s: null pointer", name);
    if (rows > (size_t(1) << 62) / cols) return fail(CTAMD_ERANGE, "%s: rows*cols overflows", name);
    size_t total = rows * cols;
    bool vec = (cols % 4 == 0) && aligned16(a) && aligned16(b) && aligned16(r) && (Op::kIn != 3 || aligned16(g));
    bool small = total < (size_t(1) << 32);
    size_t blocks = (total / 4 + size_t(kThreads) * kUnroll - 1) / (size_t(kThreads) * kUnroll);
    if (blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: more than 2^43 elements", name);
    unsigned grid = vec ? unsigned(blocks) : stream_grid(total, size_t(kThreads) * kUnroll);
    hipStream_t s = as_stream(stream);
    const int hint = hint_level(total * sizeof(float) * 2, total * sizeof(float));
    if (vec && small && hint == 2)
        hipLaunchKernelGGL((rowbcast_kernel<Op, true, uint32_t, 2>), dim3(grid), dim3(kThreads), 0, s, a, b, g, r, total, uint32_t(cols));
    else if (vec && small && hint == 1)
        hipLaunchKernelGGL((rowbcast_kernel<Op, true, uint32_t, 1>), dim3(grid), dim3(kThreads), 0, s, a, b, g, r, total, uint32_t(cols));
    else if (vec && small)
        hipLaunchKernelGGL((rowbcast_kernel<Op, true, uint32_t, 0>), dim3(grid), dim3(kThreads), 0, s, a, b, g, r, total, uint32_t(cols));
    else if (vec)
        hipLaunchKernelGGL((rowbcast_kernel<Op, true, uint64_t, 2>), dim3(grid), dim3(kThreads), 0, s, a, b, g, r, total, uint64_t(cols));
    else if (small)
        hipLaunchKernelGGL((rowbcast_kernel<Op, false, uint32_t, 0>), dim3(grid), dim3(kThreads), 0, s, a, b, g, r, total, uint32_t(cols));
    else
        hipLaunchKernelGGL((rowbcast_kernel<Op, false, uint64_t, 0>), dim3(grid), dim3(kThreads), 0, s, a, b, g, r, total, uint64_t(cols));
    account((Op::kIn == 3 ? 12.0 : 8.0) * double(total) + 4.0 * double(cols), 0.0);
    return launched(name);
}

template <class F>
int binary(const char* name, const float* a, const float* b, float* r, size_t n, void* stream) {
    Ptrs<2> in{{a, b}};
    return launch_map<F>(name, in, r, n, F(), stream);
}
template <class F>
int unary(const char* name, const float* a, float* r, size_t n, void* stream) {
    Ptrs<1> in{{a}};
    return launch_map<F>(name, in, r, n, F(), stream);
}
template <class Op>
int host_scalar(const char* name, const float* a, float s, float* r, size_t n, void* stream) {
    Ptrs<1> in{{a}};
    return launch_map<ScalarF<Op>>(name, in, r, n, ScalarF<Op>{s}, stream);
}
template <class Op>
int dev_scalar(const char* name, const float* a, const float* b1, float* r, size_t n, void* stream) {
    if (n && !b1) return fail(CTAMD_EINVAL, "%s: null scalar operand", name);
    Ptrs<1> in{{a}};
    return launch_map<DevScalarF<Op>>(name, in, r, n, DevScalarF<Op>{b1}, stream);
}


// ---- elementwise comparisons: float in, one byte (0 / 1) per element out
__device__ __forceinline__ bool compare(int cmp, float a, float b) {
    switch (cmp) {
        case CTAMD_CMP_GT: return a > b;
        case CTAMD_CMP_LT: return a < b;
        case CTAMD_CMP_EQ: return a == b;
        case CTAMD_CMP_GE: return a >= b;
        case CTAMD_CMP_LE: return a <= b;
        default: return a != b;
    }
}
// VEC: a (and b) 16-byte aligned, out 4-byte aligned: a thread compares 128-bit vectors and stores
// their four result bytes as one 32-bit word (four vectors per thread, loaded before first use);
// the last n % 4 elements and unaligned tensors go element by element.  b == nullptr: compare with s.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void compare_kernel(const float* __restrict__ a, const float* __restrict__ b, float s,
                                                           uint8_t* __restrict__ out, size_t n, int cmp) {
    if (VEC) {
        const size_t n4 = n >> 2;
        const size_t base = size_t(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
        v4f va[kUnroll], vb[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            size_t i = base + size_t(u) * kThreads;
            if (i < n4) {
                va[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(a) + i);
                if (b) vb[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(b) + i);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            size_t i = base + size_t(u) * kThreads;
            if (i < n4) {
                uint32_t word = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) word |= uint32_t(compare(cmp, va[u][e], b ? vb[u][e] : s)) << (8 * e);
                reinterpret_cast<uint32_t*>(out)[i] = word;
            }
        }
        if (blockIdx.x == 0) {
            size_t i = (n4 << 2) + threadIdx.x;
            if (i < n) out[i] = uint8_t(compare(cmp, a[i], b ? b[i] : s));
        }
    } else {
        const size_t stride = size_t(gridDim.x) * kThreads;
        for (size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride)
            out[i] = uint8_t(compare(cmp, a[i], b ? b[i] : s));
    }
}

int launch_compare(const char* name, int cmp, const float* a, const float* b, float s, uint8_t* out, size_t n, void* stream) {
    if (cmp < CTAMD_CMP_GT || cmp > CTAMD_CMP_NE) return fail(CTAMD_EINVAL, "%s: unknown comparison %d", name, cmp);
    if (n == 0) return CTAMD_OK;
    if (!a || !out) return fail(CTAMD_EINVAL, "%s: null pointer", name);
    const bool vec = aligned16(a) && (!b || aligned16(b)) && (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
    if (vec) {
        size_t blocks = (n / 4 + size_t(kThreads) * kUnroll - 1) / (size_t(kThreads) * kUnroll);
        if (blocks < 1) blocks = 1;
        if (blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: more than 2^43 elements", name);
        hipLaunchKernelGGL(compare_kernel<true>, dim3(unsigned(blocks)), dim3(kThreads), 0, as_stream(stream), a, b, s, out, n, cmp);
    } else {
        hipLaunchKernelGGL(compare_kernel<false>, dim3(stream_grid(n, kThreads)), dim3(kThreads), 0, as_stream(stream), a, b, s, out, n, cmp);
    }
    account((b ? 9.0 : 5.0) * double(n), 0.0);
    return launched(name);
}

// ---- the optimiser update of several tensors in one launch
constexpr int kSgdMaxTensors = 32;
constexpr int kSgdChunk = kThreads * 8;          // elements per block
struct SgdBatch {
    float* param[kSgdMaxTensors];
    const float* grad[kSgdMaxTensors];
    unsigned count[kSgdMaxTensors];
    unsigned first_block[kSgdMaxTensors + 1];    // block range of tensor t: [first_block[t], first_block[t+1])
    int tensors;
    float lr;
};
// param -= (0 + grad) * lr, the three operations rounded one by one.  "0 +" is what reading a
// gradient from the reference's tape does (a zero-filled buffer that contributions are added to,
// src/AutoDiff.cpp:1870-1907): it turns a -0 gradient into +0, which matters to the sign of a
// zero parameter only.
__global__ __launch_bounds__(kThreads) void sgd_multi_kernel(SgdBatch b) {
    int t = 0;
    while (t + 1 < b.tensors && blockIdx.x >= b.first_block[t + 1]) ++t;
    const unsigned begin = (blockIdx.x - b.first_block[t]) * unsigned(kSgdChunk);
    float* __restrict__ p = b.param[t];
    const float* __restrict__ g = b.grad[t];
    const unsigned n = b.count[t];
#pragma unroll
    for (int u = 0; u < kSgdChunk / kThreads; ++u) {
        unsigned i = begin + unsigned(u) * kThreads + threadIdx.x;
        if (i < n) {
            float step = (0.0f + g[i]) * b.lr;
            p[i] = p[i] - step;
        }
    }
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_add_f32(const float* a, const float* b, float* r, size_t n, void* s) { return binary<AddF>(__func__, a, b, r, n, s); }
int ctamd_sub_f32(const float* a, const float* b, float* r, size_t n, void* s) { return binary<SubF>(__func__, a, b, r, n, s); }
int ctamd_mul_f32(const float* a, const float* b, float* r, size_t n, void* s) { return binary<MulF>(__func__, a, b, r, n, s); }
int ctamd_div_f32(const float* a, const float* b, float* r, size_t n, void* s) { return binary<DivF>(__func__, a, b, r, n, s); }

int ctamd_add_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* s) {
    return launch_rowbcast<AddF>(__func__, a, b, r, rows, cols, s);
}
int ctamd_sub_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* s) {
    return launch_rowbcast<SubF>(__func__, a, b, r, rows, cols, s);
}
int ctamd_mul_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* s) {
    return launch_rowbcast<MulF>(__func__, a, b, r, rows, cols, s);
}
int ctamd_div_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* s) {
    return launch_rowbcast<DivF>(__func__, a, b, r, rows, cols, s);
}

int ctamd_add_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* s) { return dev_scalar<AddF>(__func__, a, b1, r, n, s); }
int ctamd_sub_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* s) { return dev_scalar<SubF>(__func__, a, b1, r, n, s); }
int ctamd_mul_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* s) { return dev_scalar<MulF>(__func__, a, b1, r, n, s); }
int ctamd_div_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* s) { return dev_scalar<DivF>(__func__, a, b1, r, n, s); }
int ctamd_rsub_ascalar_f32(const float* a1, const float* b, float* r, size_t n, void* s) {
    if (n && !a1) return fail(CTAMD_EINVAL, "%s: null scalar operand", __func__);
    Ptrs<1> in{{b}};
    return launch_map<RSubDevScalarF>(__func__, in, r, n, RSubDevScalarF{a1}, s);
}

int ctamd_add_scalar_f32(const float* a, float v, float* r, size_t n, void* s) { return host_scalar<AddF>(__func__, a, v, r, n, s); }
int ctamd_mul_scalar_f32(const float* a, float v, float* r, size_t n, void* s) { return host_scalar<MulF>(__func__, a, v, r, n, s); }
int ctamd_div_scalar_f32(const float* a, float v, float* r, size_t n, void* s) {
    Ptrs<1> in{{a}};
    return launch_map<DivByRcpF>(__func__, in, r, n, DivByRcpF{1.0 / double(v)}, s);
}

int ctamd_neg_f32(const float* a, float* r, size_t n, void* s) { return unary<NegF>(__func__, a, r, n, s); }
int ctamd_relu_f32(const float* a, float* r, size_t n, void* s) { return unary<ReluF>(__func__, a, r, n, s); }
int ctamd_sin_f32(const float* a, float* r, size_t n, void* s) { return unary<SinF>(__func__, a, r, n, s); }
int ctamd_cos_f32(const float* a, float* r, size_t n, void* s) { return unary<CosF>(__func__, a, r, n, s); }
int ctamd_tanh_f32(const float* a, float* r, size_t n, void* s) { return unary<TanhF>(__func__, a, r, n, s); }
int ctamd_sigmoid_f32(const float* a, float* r, size_t n, void* s) { return unary<SigmoidF>(__func__, a, r, n, s); }

int ctamd_sub_scalar_f32(const float* a, float v, float* r, size_t n, void* s) { return host_scalar<SubF>(__func__, a, v, r, n, s); }
int ctamd_abs_f32(const float* a, float* r, size_t n, void* s) { return unary<AbsF>(__func__, a, r, n, s); }
int ctamd_exp_f32(const float* a, float* r, size_t n, void* s) { return unary<ExpF>(__func__, a, r, n, s); }
int ctamd_log_f32(const float* a, float* r, size_t n, void* s) { return unary<LogF>(__func__, a, r, n, s); }
int ctamd_sqrt_f32(const float* a, float* r, size_t n, void* s) { return unary<SqrtF>(__func__, a, r, n, s); }
int ctamd_square_f32(const float* a, float* r, size_t n, void* s) { return unary<SquareF>(__func__, a, r, n, s); }
int ctamd_tan_f32(const float* a, float* r, size_t n, void* s) { return unary<TanF>(__func__, a, r, n, s); }
int ctamd_leaky_relu_f32(const float* a, float slope, float* r, size_t n, void* s) {
    Ptrs<1> in{{a}};
    return launch_map<LeakyReluF>(__func__, in, r, n, LeakyReluF{slope}, s);
}
int ctamd_abs_backward_f32(const float* x, const float* g, float* dx, size_t n, void* s) { return binary<AbsBwdF>(__func__, x, g, dx, n, s); }
int ctamd_sqrt_backward_f32(const float* y, const float* g, float* dx, size_t n, void* s) { return binary<SqrtBwdF>(__func__, y, g, dx, n, s); }
int ctamd_square_backward_f32(const float* x, const float* g, float* dx, size_t n, void* s) { return binary<SquareBwdF>(__func__, x, g, dx, n, s); }
int ctamd_tan_backward_f32(const float* y, const float* g, float* dx, size_t n, void* s) { return binary<TanBwdF>(__func__, y, g, dx, n, s); }
int ctamd_leaky_relu_backward_f32(const float* x, const float* g, float slope, float* dx, size_t n, void* s) {
    Ptrs<2> in{{x, g}};
    return launch_map<LeakyReluBwdF>(__func__, in, dx, n, LeakyReluBwdF{slope}, s);
}

int ctamd_fill_f32(float* r, float v, size_t n, void* s) {
    Ptrs<0> in{};
    return launch_map<FillF>(__func__, in, r, n, FillF{v}, s);
}
int ctamd_fill_from_f32(float* r, const float* v1, size_t n, void* s) {
    if (n && !v1) return fail(CTAMD_EINVAL, "%s: null source", __func__);
    Ptrs<0> in{};
    return launch_map<FillFromF>(__func__, in, r, n, FillFromF{v1}, s);
}
int ctamd_accumulate_f32(float* grad, const float* val, size_t n, void* s) {
    return binary<AddF>(__func__, grad, val, grad, n, s);
}
int ctamd_sgd_step_f32(float* param, const float* grad, float lr, size_t n, void* s) {
    Ptrs<2> in{{param, grad}};
    return launch_map<SgdF>(__func__, in, param, n, SgdF{lr}, s);
}
int ctamd_compare_f32(int cmp, const float* a, const float* b, uint8_t* out, size_t n, void* stream) {
    if (n && !b) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    return launch_compare(__func__, cmp, a, b, 0.0f, out, n, stream);
}
int ctamd_compare_scalar_f32(int cmp, const float* a, float s, uint8_t* out, size_t n, void* stream) {
    return launch_compare(__func__, cmp, a, nullptr, s, out, n, stream);
}
int ctamd_sgd_step_multi_f32(float* const* params, const float* const* grads, const size_t* counts, int tensors, float lr,
                             void* stream) {
    if (tensors < 0) return fail(CTAMD_EINVAL, "%s: negative tensor count", __func__);
    if (tensors && (!params || !grads || !counts)) return fail(CTAMD_EINVAL, "%s: null table", __func__);
    hipStream_t s = as_stream(stream);
    for (int done = 0; done < tensors;) {
        SgdBatch b;
        b.tensors = 0;
        b.lr = lr;
        b.first_block[0] = 0;
        double bytes = 0;
        while (done < tensors && b.tensors < kSgdMaxTensors) {
            const size_t n = counts[done];
            if (n > 0xffffffffu - unsigned(kSgdChunk)) return fail(CTAMD_ERANGE, "%s: tensor too large", __func__);
            if (n && (!params[done] || !grads[done])) return fail(CTAMD_EINVAL, "%s: null tensor", __func__);
            if (n) {
                const int t = b.tensors++;
                b.param[t] = params[done];
                b.grad[t] = grads[done];
                b.count[t] = unsigned(n);
                b.first_block[t + 1] = b.first_block[t] + unsigned((n + kSgdChunk - 1) / kSgdChunk);
                bytes += 12.0 * double(n);
            }
            ++done;
        }
        if (!b.tensors) continue;
        account(bytes, 0.0);
        hipLaunchKernelGGL(sgd_multi_kernel, dim3(b.first_block[b.tensors]), dim3(kThreads), 0, s, b);
        int rc = launched(__func__);
        if (rc) return rc;
    }
    return CTAMD_OK;
}
int ctamd_relu_backward_f32(const float* x, const float* g, float* dx, size_t n, void* s) { return binary<ReluBwdF>(__func__, x, g, dx, n, s); }
int ctamd_sigmoid_backward_f32(const float* x, const float* g, float* dx, size_t n, void* s) { return binary<SigmoidBwdF>(__func__, x, g, dx, n, s); }
int ctamd_tanh_backward_f32(const float* x, const float* g, float* dx, size_t n, void* s) { return binary<TanhBwdF>(__func__, x, g, dx, n, s); }
int ctamd_sin_backward_f32(const float* x, const float* g, float* dx, size_t n, void* s) { return binary<SinBwdF>(__func__, x, g, dx, n, s); }
int ctamd_cos_backward_f32(const float* x, const float* g, float* dx, size_t n, void* s) { return binary<CosBwdF>(__func__, x, g, dx, n, s); }
int ctamd_mse_backward_f32(const float* p, const float* t, const float* g1, float* dp, size_t n, void* s) {
    if (n && !g1) return fail(CTAMD_EINVAL, "%s: null upstream gradient", __func__);
    Ptrs<2> in{{p, t}};
    return launch_map<MseBwdF>(__func__, in, dp, n, MseBwdF{1.0 / double(float(n)), g1}, s);
}
int ctamd_mae_backward_f32(const float* p, const float* t, const float* g1, float* dp, size_t n, void* s) {
    if (n && !g1) return fail(CTAMD_EINVAL, "%s: null upstream gradient", __func__);
    Ptrs<2> in{{p, t}};
    return launch_map<MaeBwdF>(__func__, in, dp, n, MaeBwdF{1.0 / double(float(n)), g1}, s);
}
// out = acc + a * b, the product rounded first (the gradient term of Mul joining a gathered gradient)
int ctamd_mul_acc_f32(const float* a, const float* b, const float* acc, float* out, size_t n, void* s) {
    Ptrs<3> in{{a, b, acc}};
    return launch_map<PlusF<MulF>>(__func__, in, out, n, PlusF<MulF>(), s);
}
// out = acc + a / b, the quotient rounded first (Div's gradient term g / b joining a gathered
// gradient); b of a's shape, or a row vector under a [rows, cols]
int ctamd_div_acc_f32(const float* a, const float* b, const float* acc, float* out, size_t n, void* s) {
    Ptrs<3> in{{a, b, acc}};
    return launch_map<PlusF<DivF>>(__func__, in, out, n, PlusF<DivF>(), s);
}
int ctamd_div_rowbcast_acc_f32(const float* a, const float* b, const float* acc, float* out, size_t rows, size_t cols, void* s) {
    return launch_rowbcast<PlusF<DivF>>(__func__, a, b, out, rows, cols, s, acc);
}
// dx = acc + (the operator's gradient term), the term rounded first
#define CTAMD_UNARY_BACKWARD_ACC(NAME, PF)                                                                              \
    int NAME(const float* x, const float* g, const float* acc, float* dx, size_t n, void* s) {                         \
        Ptrs<3> in{{x, g, acc}};                                                                                       \
        return launch_map<PF>(__func__, in, dx, n, PF(), s);                                                           \
    }
CTAMD_UNARY_BACKWARD_ACC(ctamd_relu_backward_acc_f32, PlusF<ReluBwdF>)
CTAMD_UNARY_BACKWARD_ACC(ctamd_sigmoid_backward_acc_f32, PlusF<SigmoidBwdF>)
CTAMD_UNARY_BACKWARD_ACC(ctamd_tanh_backward_acc_f32, PlusF<TanhBwdF>)
CTAMD_UNARY_BACKWARD_ACC(ctamd_sin_backward_acc_f32, PlusRareF<SinBwdF>)
CTAMD_UNARY_BACKWARD_ACC(ctamd_cos_backward_acc_f32, PlusRareF<CosBwdF>)
#undef CTAMD_UNARY_BACKWARD_ACC
int ctamd_mse_backward_acc_f32(const float* p, const float* t, const float* g1, const float* acc, float* dp, size_t n, void* s) {
    if (n && !g1) return fail(CTAMD_EINVAL, "%s: null upstream gradient", __func__);
    Ptrs<3> in{{p, t, acc}};
    return launch_map<PlusF<MseBwdF>>(__func__, in, dp, n, PlusF<MseBwdF>{MseBwdF{1.0 / double(float(n)), g1}}, s);
}
int ctamd_mae_backward_acc_f32(const float* p, const float* t, const float* g1, const float* acc, float* dp, size_t n, void* s) {
    if (n && !g1) return fail(CTAMD_EINVAL, "%s: null upstream gradient", __func__);
    Ptrs<3> in{{p, t, acc}};
    return launch_map<PlusF<MaeBwdF>>(__func__, in, dp, n, PlusF<MaeBwdF>{MaeBwdF{1.0 / double(float(n)), g1}}, s);
}
int ctamd_div_backward_b_rowbcast_f32(const float* a, const float* b, const float* g, float* db, size_t rows, size_t cols,
                                      void* s) {
    return launch_rowbcast<DivBwdBF>(__func__, a, b, db, rows, cols, s, g);
}
int ctamd_div_backward_b_f32(const float* a, const float* b, const float* g, float* db, size_t n, void* s) {
    Ptrs<3> in{{a, b, g}};
    return launch_map<DivBwdBF>(__func__, in, db, n, DivBwdBF(), s);
}

}  // extern "C"
