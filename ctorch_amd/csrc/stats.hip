// Reductions along one axis and their gradients: sum, mean, max, min, var, std of a tensor viewed
// as [outer, len, inner] (row-major) over its middle axis.  outer = inner = 1 is the reduction of a
// whole tensor; inner = 1 reduces the rows of a matrix, outer = 1 its columns.  These are the
// methods the reference declares on Tensor without defining them (include/Tensor.h:824-948); the
// arithmetic is fixed here and restated by the CPU oracle:
//   sum, mean   fp32 terms, added in a tree (double across threads); mean = float(sum) / float(len)
//   max, min    the extreme value and the position of its first occurrence (NaN never wins unless it
//               is the first element, as a loop `if (v > m) m = v` that starts from element 0 behaves)
//   var, std    sums of (x - K) and (x - K)^2 in double about K = the first element of the run (the
//               shift keeps the cancellation in s2 - s1^2 / n harmless), divisor len - ddof
// All kernels are HBM-bound streams (4 bytes per element forward): 128-bit loads, four in flight per
// thread.  A run that must be shared by several blocks to fill the chip is cut into chunks whose
// partial results (16 bytes each, in the per-device scratch) a second launch merges in a fixed order.
#include "common.h"
#include "devmath.h"

namespace ctamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;
constexpr int kInFlight = 4;

enum Kind { kSum = CTAMD_RED_SUM, kMean = CTAMD_RED_MEAN, kMax = CTAMD_RED_MAX, kMin = CTAMD_RED_MIN,
            kVar = CTAMD_RED_VAR, kStd = CTAMD_RED_STD };

// A partial result: (sum, -) | (value, position) | (s1, s2).  A float value and a position below
// 2^31 are exact in a double, so one layout serves every kind.
struct Part {
    double a, b;
};
constexpr double kNoPos = 2147483648.0;   // "no element yet": larger than any position

template <int KIND>
__device__ __forceinline__ Part empty_part() {
    if (KIND == kMax) return Part{-__builtin_huge_val(), kNoPos};
    if (KIND == kMin) return Part{__builtin_huge_val(), kNoPos};
    return Part{0.0, 0.0};
}
// Associative and commutative (ties go to the smaller position), so any merge order gives the same
// extreme; sums are merged in a fixed order by construction of the callers.
template <int KIND>
__device__ __forceinline__ Part merge(Part p, Part o) {
    const double pa = p.a, pb = p.b, oa = o.a, ob = o.b;       // by value: selects on registers, not on addresses
    if (KIND == kMax || KIND == kMin) {
        const bool better = (KIND == kMax) ? (oa > pa) : (oa < pa);
        const bool take = better || (oa == pa && ob < pb);
        Part r;
        r.a = take ? oa : pa;
        r.b = take ? ob : pb;
        return r;
    }
    return Part{pa + oa, pb + ob};
}
template <int KIND>
__device__ __forceinline__ Part wave_merge(Part p) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        Part o{__shfl_xor(p.a, off, 64), __shfl_xor(p.b, off, 64)};
        p = merge<KIND>(p, o);
    }
    return p;
}

// Per-thread running state.  Sums keep fp32 lanes (converted to double once at the end); var / std
// two double chains per sum.
template <int KIND>
struct Local {
    float f[8];
    double d[4];
    float best;
    unsigned pos;
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) d[i] = 0.0;
        best = (KIND == kMax) ? -__builtin_huge_valf() : __builtin_huge_valf();
        pos = 0x80000000u;
    }
    // element v at position p of its run; `lane` (0..7) spreads independent accumulators
    __device__ __forceinline__ void take(float v, unsigned p, int lane, double shift) {
        if (KIND == kSum || KIND == kMean) {
            f[lane & 7] += v;
        } else if (KIND == kMax) {
            const bool up = v > best;
            best = up ? v : best;
            pos = up ? p : pos;
        } else if (KIND == kMin) {
            const bool up = v < best;
            best = up ? v : best;
            pos = up ? p : pos;
        } else {
            const double t = double(v) - shift;
            d[lane & 1] += t;
            d[2 + (lane & 1)] = __fma_rn(t, t, d[2 + (lane & 1)]);
        }
    }
    __device__ __forceinline__ Part part() const {
        if (KIND == kSum || KIND == kMean) {
            double t = ((double(f[0]) + double(f[1])) + (double(f[2]) + double(f[3]))) +
                       ((double(f[4]) + double(f[5])) + (double(f[6]) + double(f[7])));
            return Part{t, 0.0};
        }
        if (KIND == kMax || KIND == kMin) return Part{double(best), pos == 0x80000000u ? kNoPos : double(pos)};
        return Part{d[0] + d[1], d[2] + d[3]};
    }
};

// The result of a run from its merged partial.  first = element 0 of the run.
template <int KIND>
__device__ __forceinline__ void finish(const Part& p, float first, size_t len, int ddof, float* out, int32_t* index,
                                       float* mean_out, size_t at) {
    if (KIND == kSum) {
        out[at] = float(p.a);
    } else if (KIND == kMean) {
        out[at] = float(p.a) / float(len);
    } else if (KIND == kMax || KIND == kMin) {
        // a NaN in front stays (nothing compares greater than it); an all -inf / +inf / NaN-free-of-winners run
        // keeps element 0
        const bool keep_first = (first != first) || p.b >= kNoPos;
        out[at] = keep_first ? first : float(p.a);
        if (index) index[at] = keep_first ? 0 : int32_t(p.b);
    } else {
        const double n = double(len);
        const double m2 = p.b - p.a * p.a / n;                 // sum of squared deviations from the mean
        double var = m2 / (n - double(ddof));                   // n == ddof: 0 / 0 = NaN, x / 0 = inf, as the formula says
        if (var < 0.0) var = 0.0;                               // rounding of a constant run
        out[at] = (KIND == kVar) ? float(var) : float(__builtin_sqrt(var));
        if (mean_out) mean_out[at] = float(double(first) + p.a / n);
    }
}

// ------------------------------------------------------------------------ contiguous axis
// inner == 1: `rows` runs of `cols` contiguous elements.  A group of GROUP threads (a wave, or the
// whole block) owns one chunk of one run.
template <int KIND, bool VEC, int GROUP>
__global__ __launch_bounds__(kThreads) void reduce_rows_kernel(const float* __restrict__ x, Part* __restrict__ parts,
                                                               float* __restrict__ out, int32_t* __restrict__ index,
                                                               float* __restrict__ mean_out, size_t rows, size_t cols,
                                                               size_t chunk_len, unsigned chunks, int ddof) {
    constexpr int kGroups = kThreads / GROUP;
    __shared__ Part s_part[kThreads / 64];
    const unsigned lane = threadIdx.x % GROUP;
    const size_t work = size_t(blockIdx.x) * kGroups + threadIdx.x / GROUP;
    const bool live = work < rows * chunks;
    const size_t row = live ? work / chunks : 0;
    const unsigned chunk = live ? unsigned(work % chunks) : 0;
    const float* __restrict__ xr = x + row * cols;
    const size_t c0 = live ? size_t(chunk) * chunk_len : 0;
    size_t c1 = live ? c0 + chunk_len : 0;
    if (c1 > cols) c1 = cols;
    const float first = xr[0];
    const double shift = double(first);
    Local<KIND> acc;
    acc.init();
    if (VEC) {
        const v4f* __restrict__ xv = reinterpret_cast<const v4f*>(xr);
        const size_t v0 = c0 >> 2, v1 = c1 >> 2;
        size_t i = v0 + lane;
        for (; i + size_t(kInFlight - 1) * GROUP < v1; i += size_t(kInFlight) * GROUP) {
            v4f v[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) v[u] = __builtin_nontemporal_load(xv + i + size_t(u) * GROUP);
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc.take(v[u][e], unsigned((i + size_t(u) * GROUP) * 4 + e), (u & 1) * 4 + e, shift);
        }
        for (; i < v1; i += GROUP) {
            const v4f v = __builtin_nontemporal_load(xv + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc.take(v[e], unsigned(i * 4 + e), e, shift);
        }
    } else {
        size_t i = c0 + lane;
        for (; i + size_t(kInFlight - 1) * GROUP < c1; i += size_t(kInFlight) * GROUP) {
            float v[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) v[u] = xr[i + size_t(u) * GROUP];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) acc.take(v[u], unsigned(i + size_t(u) * GROUP), u, shift);
        }
        for (; i < c1; i += GROUP) acc.take(xr[i], unsigned(i), 0, shift);
    }
    Part p = wave_merge<KIND>(acc.part());
    if (GROUP > 64) {
        if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = p;
        __syncthreads();
        if (threadIdx.x == 0) {
            p = s_part[0];
#pragma unroll
            for (int w = 1; w < kThreads / 64; ++w) p = merge<KIND>(p, s_part[w]);
        }
    }
    if (lane == 0 && live) {
        if (chunks == 1) finish<KIND>(p, first, cols, ddof, out, index, mean_out, row);
        else parts[work] = p;
    }
}

// ----------------------------------------------------------------------------- strided axis
// inner > 1: for each of `outer` slabs, a [len, inner] matrix whose rows are folded.  A block's
// threads form TY = 256 / tx_count row groups of tx_count lanes; a lane owns W adjacent columns and
// its group walks rows ty, ty + TY, ... of the block's chunk, four rows in flight.  The groups are
// merged through LDS in group order.
template <int KIND, int W>
__global__ __launch_bounds__(kThreads) void reduce_cols_kernel(const float* __restrict__ x, Part* __restrict__ parts,
                                                               float* __restrict__ out, int32_t* __restrict__ index,
                                                               float* __restrict__ mean_out, size_t len, size_t inner,
                                                               size_t rows_per_chunk, unsigned chunks, unsigned tx_count,
                                                               int ddof) {
    __shared__ Part s_part[kThreads * W];
    const unsigned tx = threadIdx.x % tx_count, ty = threadIdx.x / tx_count, ty_count = kThreads / tx_count;
    const size_t col = (size_t(blockIdx.x) * tx_count + tx) * W;
    const bool live = col < inner;
    const float* __restrict__ slab = x + size_t(blockIdx.z) * len * inner;
    const size_t r0 = size_t(blockIdx.y) * rows_per_chunk;
    size_t r1 = r0 + rows_per_chunk;
    if (r1 > len) r1 = len;
    Local<KIND> acc[W];
    float first[W];
    double shift[W];
#pragma unroll
    for (int e = 0; e < W; ++e) {
        acc[e].init();
        first[e] = live ? slab[col + e] : 0.0f;
        shift[e] = double(first[e]);
    }
    if (live) {
        auto load = [&](size_t r, float (&v)[W]) {
            if (W == 4) {
                const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(slab + r * inner + col));
#pragma unroll
                for (int e = 0; e < W; ++e) v[e] = t[e];
            } else {
                v[0] = slab[r * inner + col];
            }
        };
        size_t r = r0 + ty;
        for (; r + size_t(kInFlight - 1) * ty_count < r1; r += size_t(kInFlight) * ty_count) {
            float v[kInFlight][W];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) load(r + size_t(u) * ty_count, v[u]);
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
#pragma unroll
                for (int e = 0; e < W; ++e) acc[e].take(v[u][e], unsigned(r + size_t(u) * ty_count), u, shift[e]);
        }
        for (; r < r1; r += ty_count) {
            float v[W];
            load(r, v);
#pragma unroll
            for (int e = 0; e < W; ++e) acc[e].take(v[e], unsigned(r), 0, shift[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < W; ++e) s_part[(ty * tx_count + tx) * W + e] = acc[e].part();
    __syncthreads();
    if (ty == 0 && live) {
#pragma unroll
        for (int e = 0; e < W; ++e) {
            Part p = s_part[tx * W + e];
            for (unsigned k = 1; k < ty_count; ++k) p = merge<KIND>(p, s_part[(k * tx_count + tx) * W + e]);
            const size_t at = size_t(blockIdx.z) * inner + col + e;
            if (chunks == 1) finish<KIND>(p, first[e], len, ddof, out, index, mean_out, at);
            else parts[(size_t(blockIdx.z) * chunks + blockIdx.y) * inner + col + e] = p;
        }
    }
}

// Second launch: the `chunks` partials of each result merged.  Contiguous axis (inner == 1): a wave
// per result, lane t takes chunks t, t + 64, ...; strided axis: a block folds 32 neighbouring
// results, its 8 groups of 32 lanes take every 8th chunk (neighbouring lanes read neighbouring
// partials) and are merged through LDS in group order.
constexpr int kFinishCols = 32, kFinishGroups = kThreads / kFinishCols;
template <int KIND, bool WAVE>
__global__ __launch_bounds__(kThreads) void reduce_finish_kernel(const Part* __restrict__ parts, const float* __restrict__ x,
                                                                 float* __restrict__ out, int32_t* __restrict__ index,
                                                                 float* __restrict__ mean_out, size_t results, size_t len,
                                                                 size_t inner, unsigned chunks, int ddof) {
    if (WAVE) {
        const size_t r = size_t(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6);
        const unsigned lane = threadIdx.x & 63;
        Part p = empty_part<KIND>();
        if (r < results)
            for (unsigned k = lane; k < chunks; k += 64) p = merge<KIND>(p, parts[r * chunks + k]);
        p = wave_merge<KIND>(p);
        if (lane == 0 && r < results) finish<KIND>(p, x[r * len], len, ddof, out, index, mean_out, r);
    } else {
        __shared__ Part s_part[kFinishGroups][kFinishCols];
        const unsigned lane = threadIdx.x % kFinishCols, group = threadIdx.x / kFinishCols;
        const size_t r = size_t(blockIdx.x) * kFinishCols + lane;
        const bool live = r < results;
        const size_t slab = live ? r / inner : 0, c = live ? r % inner : 0;
        Part p = empty_part<KIND>();
        if (live) {
            unsigned k = group;
            for (; k + 3 * kFinishGroups < chunks; k += 4 * kFinishGroups) {
                Part q[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) q[u] = parts[(slab * chunks + k + u * kFinishGroups) * inner + c];
#pragma unroll
                for (int u = 0; u < 4; ++u) p = merge<KIND>(p, q[u]);
            }
            for (; k < chunks; k += kFinishGroups) p = merge<KIND>(p, parts[(slab * chunks + k) * inner + c]);
        }
        s_part[group][lane] = p;
        __syncthreads();
        if (group == 0 && live) {
#pragma unroll
            for (int g = 1; g < kFinishGroups; ++g) p = merge<KIND>(p, s_part[g][lane]);
            finish<KIND>(p, x[slab * len * inner + c], len, ddof, out, index, mean_out, r);
        }
    }
}

// ----------------------------------------------------------------------------- gradients
// What one result passes to every element of its run.
struct Upstream {
    float g, aux, y;     // upstream gradient; mean (var / std); result (std)
    int32_t pos;         // position of the extreme element (max / min)
    double rcp;          // 1 / divisor of the run (mean: len; var: len - ddof; std: (len - ddof) * y)
};
template <int KIND>
__device__ __forceinline__ Upstream upstream(const float* y, const int32_t* index, const float* mean, const float* g, size_t at,
                                             size_t len, int ddof) {
    Upstream u{g[at], 0.0f, 0.0f, 0, 0.0};
    if (KIND == kMean) u.rcp = 1.0 / double(float(len));
    if (KIND == kMax || KIND == kMin) u.pos = index[at];
    if (KIND == kVar || KIND == kStd) {
        u.aux = mean[at];
        const float nf = float(double(len) - double(ddof));
        if (KIND == kVar) u.rcp = 1.0 / double(nf);
        else {
            u.y = y[at];
            u.rcp = 1.0 / double(nf * u.y);
        }
    }
    return u;
}
// fp32 operation order (the oracle's): sum g; mean g / float(len); max / min the gradient at the
// extreme's position and +0 elsewhere; var ((x - mean) * 2 / float(len - ddof)) * g; std
// ((x - mean) / (float(len - ddof) * y)) * g.  Divisions by a run's divisor go through its double
// reciprocal (the exact fp32 quotient).
template <int KIND>
__device__ __forceinline__ float grad_one(const Upstream& u, float xv, unsigned p) {
    if (KIND == kSum) return u.g;
    if (KIND == kMean) return cta_div_rcp(u.g, u.rcp);
    if (KIND == kMax || KIND == kMin) return (int32_t(p) == u.pos) ? u.g : 0.0f;
    const float d = xv - u.aux;
    if (KIND == kVar) {
        const float t = d * 2.0f;
        return cta_div_rcp(t, u.rcp) * u.g;
    }
    return cta_div_rcp(d, u.rcp) * u.g;
}
template <int KIND>
constexpr bool reads_x() { return KIND == kVar || KIND == kStd; }

template <int KIND, bool VEC, int GROUP>
__global__ __launch_bounds__(kThreads) void reduce_rows_backward_kernel(const float* __restrict__ x, const float* __restrict__ y,
                                                                        const int32_t* __restrict__ index, const float* __restrict__ mean,
                                                                        const float* __restrict__ g, float* __restrict__ dx, size_t rows,
                                                                        size_t cols, size_t chunk_len, unsigned chunks, int ddof) {
    constexpr int kGroups = kThreads / GROUP;
    const unsigned lane = threadIdx.x % GROUP;
    const size_t work = size_t(blockIdx.x) * kGroups + threadIdx.x / GROUP;
    if (work >= rows * chunks) return;
    const size_t row = work / chunks;
    const size_t c0 = size_t(work % chunks) * chunk_len;
    size_t c1 = c0 + chunk_len;
    if (c1 > cols) c1 = cols;
    const Upstream u = upstream<KIND>(y, index, mean, g, row, cols, ddof);
    const float* __restrict__ xr = reads_x<KIND>() ? x + row * cols : nullptr;
    float* __restrict__ dr = dx + row * cols;
    if (VEC) {
        const size_t v1 = c1 >> 2;
        size_t i = (c0 >> 2) + lane;
        for (; i + size_t(kInFlight - 1) * GROUP < v1; i += size_t(kInFlight) * GROUP) {
            v4f v[kInFlight];
            if (reads_x<KIND>()) {
#pragma unroll
                for (int k = 0; k < kInFlight; ++k) v[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(xr) + i + size_t(k) * GROUP);
            }
#pragma unroll
            for (int k = 0; k < kInFlight; ++k) {
                v4f o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = grad_one<KIND>(u, reads_x<KIND>() ? v[k][e] : 0.0f, unsigned((i + size_t(k) * GROUP) * 4 + e));
                __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(dr) + i + size_t(k) * GROUP);
            }
        }
        for (; i < v1; i += GROUP) {
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f}, o;
            if (reads_x<KIND>()) v = reinterpret_cast<const v4f*>(xr)[i];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = grad_one<KIND>(u, v[e], unsigned(i * 4 + e));
            reinterpret_cast<v4f*>(dr)[i] = o;
        }
    } else {
        for (size_t i = c0 + lane; i < c1; i += GROUP) dr[i] = grad_one<KIND>(u, reads_x<KIND>() ? xr[i] : 0.0f, unsigned(i));
    }
}

template <int KIND, int W>
__global__ __launch_bounds__(kThreads) void reduce_cols_backward_kernel(const float* __restrict__ x, const float* __restrict__ y,
                                                                        const int32_t* __restrict__ index, const float* __restrict__ mean,
                                                                        const float* __restrict__ g, float* __restrict__ dx, size_t len,
                                                                        size_t inner, size_t rows_per_chunk, unsigned tx_count, int ddof) {
    const unsigned tx = threadIdx.x % tx_count, ty = threadIdx.x / tx_count, ty_count = kThreads / tx_count;
    const size_t col = (size_t(blockIdx.x) * tx_count + tx) * W;
    if (col >= inner) return;
    const size_t slab_at = size_t(blockIdx.z) * len * inner;
    const size_t r0 = size_t(blockIdx.y) * rows_per_chunk;
    size_t r1 = r0 + rows_per_chunk;
    if (r1 > len) r1 = len;
    Upstream u[W];
#pragma unroll
    for (int e = 0; e < W; ++e) u[e] = upstream<KIND>(y, index, mean, g, size_t(blockIdx.z) * inner + col + e, len, ddof);
    auto one_row = [&](size_t r, const float (&v)[W]) {
        float o[W];
#pragma unroll
        for (int e = 0; e < W; ++e) o[e] = grad_one<KIND>(u[e], v[e], unsigned(r));
        float* dst = dx + slab_at + r * inner + col;
        if (W == 4) {
            v4f t = {o[0], o[1 % W], o[2 % W], o[3 % W]};
            __builtin_nontemporal_store(t, reinterpret_cast<v4f*>(dst));
        } else {
            dst[0] = o[0];
        }
    };
    size_t r = r0 + ty;
    for (; r + size_t(kInFlight - 1) * ty_count < r1; r += size_t(kInFlight) * ty_count) {
        float v[kInFlight][W] = {};
        if (reads_x<KIND>()) {
#pragma unroll
            for (int k = 0; k < kInFlight; ++k) {
                const float* src = x + slab_at + (r + size_t(k) * ty_count) * inner + col;
                if (W == 4) {
                    const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src));
#pragma unroll
                    for (int e = 0; e < W; ++e) v[k][e] = t[e];
                } else {
                    v[k][0] = src[0];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) one_row(r + size_t(k) * ty_count, v[k]);
    }
    for (; r < r1; r += ty_count) {
        float v[W] = {};
        if (reads_x<KIND>()) {
#pragma unroll
            for (int e = 0; e < W; ++e) v[e] = x[slab_at + r * inner + col + e];
        }
        one_row(r, v);
    }
}

// ------------------------------------------------------------------------------- launch plans
struct RowPlan {
    size_t chunk_len;
    unsigned chunks;
    int group;
    bool vec;
    unsigned grid;
};
// `want_chunks`: whether a run may be shared by several blocks (forward; the gradient has no merge
// step, its chunks only spread the work).
bool plan_rows(const float* x, const void* other, size_t rows, size_t cols, RowPlan& p) {
    const size_t target = size_t(compute_units() > 0 ? compute_units() : 256) * 4;
    p.vec = cols % 4 == 0 && aligned16(x) && (!other || aligned16(other));
    size_t chunks = 1;
    if (rows < target) {
        chunks = (target + rows - 1) / rows;
        const size_t most = (cols + 4095) / 4096;           // a chunk is at least 4096 elements
        if (chunks > most) chunks = most;
        if (chunks > 2048) chunks = 2048;
        if (chunks < 1) chunks = 1;
    }
    p.chunk_len = ((cols + chunks - 1) / chunks + 3) & ~size_t(3);
    chunks = (cols + p.chunk_len - 1) / p.chunk_len;
    p.chunks = unsigned(chunks);
    p.group = p.chunk_len <= 1024 ? 64 : 256;
    const size_t work = rows * chunks, per_block = size_t(kThreads / p.group);
    const size_t blocks = (work + per_block - 1) / per_block;
    if (blocks > 0x7fffffffu) return false;
    p.grid = unsigned(blocks);
    return true;
}
struct ColPlan {
    size_t rows_per_chunk;
    unsigned chunks, tx_count;
    bool vec;
    dim3 grid;
};
constexpr size_t kMaxGridZ = 65535;
bool plan_cols(const float* x, const void* other, size_t outer, size_t len, size_t inner, ColPlan& p) {
    const size_t target = size_t(compute_units() > 0 ? compute_units() : 256) * 4;
    p.vec = inner % 4 == 0 && aligned16(x) && (!other || aligned16(other));
    const size_t w = p.vec ? 4 : 1;
    const size_t lanes = (inner + w - 1) / w;
    unsigned tx = 4;
    while (tx < kThreads && tx < lanes) tx <<= 1;
    p.tx_count = tx;
    const size_t ty = kThreads / tx;
    const size_t strips = (lanes + tx - 1) / tx;
    size_t chunks = 1;
    if (strips * outer < target) {
        chunks = (target + strips * outer - 1) / (strips * outer);
        const size_t most = (len + ty * 8 - 1) / (ty * 8);    // a chunk gives every row group eight rows
        if (chunks > most) chunks = most;
        if (chunks > 256) chunks = 256;
        if (chunks < 1) chunks = 1;
    }
    p.rows_per_chunk = (len + chunks - 1) / chunks;
    chunks = (len + p.rows_per_chunk - 1) / p.rows_per_chunk;
    p.chunks = unsigned(chunks);
    if (strips > 0x7fffffffu || chunks > 65535) return false;
    // the grid's third dimension holds at most kMaxGridZ slabs: a launch per run of that many (p.grid.z is the first run's)
    p.grid = dim3(unsigned(strips), unsigned(chunks), unsigned(outer < kMaxGridZ ? outer : kMaxGridZ));
    return true;
}
template <class T>
T* at_offset(T* p, size_t n) { return p ? p + n : nullptr; }

template <int KIND>
int run_forward(const char* name, const float* x, float* out, int32_t* index, float* mean_out, size_t outer, size_t len,
                size_t inner, int ddof, hipStream_t s) {
    ScratchUse use(static_cast<void*>(s));
    Part* parts = reinterpret_cast<Part*>(use.ptr());
    if (!parts) return CTAMD_EINVAL;
    constexpr size_t kSlots = kScratchFloats * sizeof(float) / sizeof(Part);
    if (inner == 1) {
        RowPlan p;
        if (!plan_rows(x, nullptr, outer, len, p)) return fail(CTAMD_ERANGE, "%s: too many runs", name);
        if (p.chunks > 1 && outer * p.chunks > kSlots) return fail(CTAMD_ERANGE, "%s: partial results exceed the scratch buffer", name);
#define CTAMD_ROWS(V, G) hipLaunchKernelGGL((reduce_rows_kernel<KIND, V, G>), dim3(p.grid), dim3(kThreads), 0, s, x, parts, out, index, \
                                            mean_out, outer, len, p.chunk_len, p.chunks, ddof)
        if (p.vec && p.group == 64) CTAMD_ROWS(true, 64);
        else if (p.vec) CTAMD_ROWS(true, 256);
        else if (p.group == 64) CTAMD_ROWS(false, 64);
        else CTAMD_ROWS(false, 256);
#undef CTAMD_ROWS
        int rc = launched(name);
        if (rc || p.chunks == 1) return rc;
        hipLaunchKernelGGL((reduce_finish_kernel<KIND, true>), dim3(unsigned((outer + 3) / 4)), dim3(kThreads), 0, s, parts, x, out, index,
                           mean_out, outer, len, size_t(1), p.chunks, ddof);
        return launched(name);
    }
    ColPlan p;
    if (!plan_cols(x, nullptr, outer, len, inner, p)) return fail(CTAMD_ERANGE, "%s: shape exceeds the launch grid", name);
    if (p.chunks > 1 && outer * p.chunks * inner > kSlots) {
        // fall back to one chunk per column strip: slower for a tall narrow slab, always fits
        p.chunks = 1;
        p.rows_per_chunk = len;
        p.grid.y = 1;
    }
    for (size_t o0 = 0; o0 < outer; o0 += kMaxGridZ) {
        p.grid.z = unsigned(outer - o0 < kMaxGridZ ? outer - o0 : kMaxGridZ);
        const float* xs = x + o0 * len * inner;
        Part* ps = parts + o0 * p.chunks * inner;
        if (p.vec)
            hipLaunchKernelGGL((reduce_cols_kernel<KIND, 4>), p.grid, dim3(kThreads), 0, s, xs, ps, at_offset(out, o0 * inner),
                               at_offset(index, o0 * inner), at_offset(mean_out, o0 * inner), len, inner, p.rows_per_chunk, p.chunks, p.tx_count, ddof);
        else
            hipLaunchKernelGGL((reduce_cols_kernel<KIND, 1>), p.grid, dim3(kThreads), 0, s, xs, ps, at_offset(out, o0 * inner),
                               at_offset(index, o0 * inner), at_offset(mean_out, o0 * inner), len, inner, p.rows_per_chunk, p.chunks, p.tx_count, ddof);
    }
    int rc = launched(name);
    if (rc || p.chunks == 1) return rc;
    const size_t results = outer * inner;
    hipLaunchKernelGGL((reduce_finish_kernel<KIND, false>), dim3(unsigned((results + kFinishCols - 1) / kFinishCols)), dim3(kThreads), 0, s, parts,
                       x, out, index, mean_out, results, len, inner, p.chunks, ddof);
    return launched(name);
}

template <int KIND>
int run_backward(const char* name, const float* x, const float* y, const int32_t* index, const float* mean, const float* g, float* dx,
                 size_t outer, size_t len, size_t inner, int ddof, hipStream_t s) {
    if (inner == 1) {
        RowPlan p;
        if (!plan_rows(reads_x<KIND>() ? x : dx, dx, outer, len, p)) return fail(CTAMD_ERANGE, "%s: too many runs", name);
#define CTAMD_ROWS(V, G) hipLaunchKernelGGL((reduce_rows_backward_kernel<KIND, V, G>), dim3(p.grid), dim3(kThreads), 0, s, x, y, index, mean, \
                                            g, dx, outer, len, p.chunk_len, p.chunks, ddof)
        if (p.vec && p.group == 64) CTAMD_ROWS(true, 64);
        else if (p.vec) CTAMD_ROWS(true, 256);
        else if (p.group == 64) CTAMD_ROWS(false, 64);
        else CTAMD_ROWS(false, 256);
#undef CTAMD_ROWS
        return launched(name);
    }
    ColPlan p;
    if (!plan_cols(reads_x<KIND>() ? x : dx, dx, outer, len, inner, p)) return fail(CTAMD_ERANGE, "%s: shape exceeds the launch grid", name);
    for (size_t o0 = 0; o0 < outer; o0 += kMaxGridZ) {
        p.grid.z = unsigned(outer - o0 < kMaxGridZ ? outer - o0 : kMaxGridZ);
        if (p.vec)
            hipLaunchKernelGGL((reduce_cols_backward_kernel<KIND, 4>), p.grid, dim3(kThreads), 0, s, at_offset(x, o0 * len * inner),
                               at_offset(y, o0 * inner), at_offset(index, o0 * inner), at_offset(mean, o0 * inner), at_offset(g, o0 * inner),
                               dx + o0 * len * inner, len, inner, p.rows_per_chunk, p.tx_count, ddof);
        else
            hipLaunchKernelGGL((reduce_cols_backward_kernel<KIND, 1>), p.grid, dim3(kThreads), 0, s, at_offset(x, o0 * len * inner),
                               at_offset(y, o0 * inner), at_offset(index, o0 * inner), at_offset(mean, o0 * inner), at_offset(g, o0 * inner),
                               dx + o0 * len * inner, len, inner, p.rows_per_chunk, p.tx_count, ddof);
    }
    return launched(name);
}

// out[i] = g[i] + g[i + n] + g[i + 2n] + ..., added in that order in fp32 from 0: the fold the
// reference's gradient shape adjustment falls back to for shapes that do not broadcast
// (src/AutoDiff.cpp:968-1046).  One thread per output element.
__global__ __launch_bounds__(kThreads) void fold_mod_kernel(const float* __restrict__ g, float* __restrict__ out, size_t g_count,
                                                            size_t out_count) {
    const size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= out_count) return;
    float sum = 0.0f;
    for (size_t j = i; j < g_count; j += out_count) sum += g[j];
    out[i] = sum;
}

// out[t] = sum of g over the dimensions in which the target's extent is 1 and the gradient's is not;
// a dimension in which the gradient's extent is 1 is repeated (stride 0).  One thread per output
// element, the summed dimensions walked in index order, in double.  The general form behind the
// gradient of a broadcast operand; the shapes that matter for speed ([rows, cols] -> [cols], one
// element) have kernels of their own.
constexpr int kMaxDims = 8;
struct BroadcastPlan {
    int rank;
    unsigned long long out_extent[kMaxDims];    // the target's extents, padded with leading 1s
    unsigned long long keep_stride[kMaxDims];   // the gradient's stride where the coordinate is kept, else 0
    unsigned long long red_extent[kMaxDims];    // the gradient's extent where it is summed over, else 1
    unsigned long long red_stride[kMaxDims];
    unsigned long long reduced;                 // product of red_extent
};
__global__ __launch_bounds__(kThreads) void broadcast_reduce_kernel(const float* __restrict__ g, float* __restrict__ out,
                                                                    size_t out_count, BroadcastPlan p) {
    const size_t o = size_t(blockIdx.x) * kThreads + threadIdx.x;
    if (o >= out_count) return;
    size_t rem = o, base = 0;
    for (int d = p.rank - 1; d >= 0; --d) {
        const size_t c = rem % p.out_extent[d];
        rem /= p.out_extent[d];
        base += c * p.keep_stride[d];
    }
    double sum = 0.0;
    for (size_t r = 0; r < p.reduced; ++r) {
        size_t q = r, at = base;
        for (int d = p.rank - 1; d >= 0; --d) {
            at += (q % p.red_extent[d]) * p.red_stride[d];
            q /= p.red_extent[d];
        }
        sum += double(g[at]);
    }
    out[o] = float(sum);
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_reduce_dim_f32(int kind, const float* x, float* out, int32_t* index, float* mean_out, size_t outer, size_t len,
                         size_t inner, int ddof, void* stream) {
    if (kind < CTAMD_RED_SUM || kind > CTAMD_RED_STD) return fail(CTAMD_EINVAL, "%s: unknown reduction %d", __func__, kind);
    if (outer == 0 || inner == 0) return CTAMD_OK;
    if (!out) return fail(CTAMD_EINVAL, "%s: null output", __func__);
    if (len == 0) return fail(CTAMD_EINVAL, "%s: reduction over an empty axis", __func__);
    if (!x) return fail(CTAMD_EINVAL, "%s: null input", __func__);
    if (len > size_t(0x7fffffff)) return fail(CTAMD_ERANGE, "%s: more than 2^31-1 elements along the axis", __func__);
    if (outer > (size_t(1) << 62) / len || outer * len > (size_t(1) << 62) / inner) return fail(CTAMD_ERANGE, "%s: shape overflows", __func__);
    hipStream_t s = as_stream(stream);
    account(4.0 * double(outer) * double(len) * double(inner) + 4.0 * double(outer) * double(inner), double(outer) * double(len) * double(inner));
    switch (kind) {
        case CTAMD_RED_SUM: return run_forward<kSum>(__func__, x, out, index, mean_out, outer, len, inner, ddof, s);
        case CTAMD_RED_MEAN: return run_forward<kMean>(__func__, x, out, index, mean_out, outer, len, inner, ddof, s);
        case CTAMD_RED_MAX: return run_forward<kMax>(__func__, x, out, index, mean_out, outer, len, inner, ddof, s);
        case CTAMD_RED_MIN: return run_forward<kMin>(__func__, x, out, index, mean_out, outer, len, inner, ddof, s);
        case CTAMD_RED_VAR: return run_forward<kVar>(__func__, x, out, index, mean_out, outer, len, inner, ddof, s);
        default: return run_forward<kStd>(__func__, x, out, index, mean_out, outer, len, inner, ddof, s);
    }
}

int ctamd_reduce_dim_backward_f32(int kind, const float* x, const float* y, const int32_t* index, const float* mean, const float* g,
                                  float* dx, size_t outer, size_t len, size_t inner, int ddof, void* stream) {
    if (kind < CTAMD_RED_SUM || kind > CTAMD_RED_STD) return fail(CTAMD_EINVAL, "%s: unknown reduction %d", __func__, kind);
    if (outer == 0 || inner == 0 || len == 0) return CTAMD_OK;
    if (!g || !dx) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    const bool extreme = kind == CTAMD_RED_MAX || kind == CTAMD_RED_MIN, spread = kind == CTAMD_RED_VAR || kind == CTAMD_RED_STD;
    if (extreme && !index) return fail(CTAMD_EINVAL, "%s: max / min need the positions the forward pass returned", __func__);
    if (spread && (!x || !mean)) return fail(CTAMD_EINVAL, "%s: var / std need the input and its mean", __func__);
    if (kind == CTAMD_RED_STD && !y) return fail(CTAMD_EINVAL, "%s: std needs its result", __func__);
    if (len > size_t(0x7fffffff)) return fail(CTAMD_ERANGE, "%s: more than 2^31-1 elements along the axis", __func__);
    if (outer > (size_t(1) << 62) / len || outer * len > (size_t(1) << 62) / inner) return fail(CTAMD_ERANGE, "%s: shape overflows", __func__);
    hipStream_t s = as_stream(stream);
    account((spread ? 8.0 : 4.0) * double(outer) * double(len) * double(inner) + 4.0 * double(outer) * double(inner), 0.0);
    switch (kind) {
        case CTAMD_RED_SUM: return run_backward<kSum>(__func__, x, y, index, mean, g, dx, outer, len, inner, ddof, s);
        case CTAMD_RED_MEAN: return run_backward<kMean>(__func__, x, y, index, mean, g, dx, outer, len, inner, ddof, s);
        case CTAMD_RED_MAX: return run_backward<kMax>(__func__, x, y, index, mean, g, dx, outer, len, inner, ddof, s);
        case CTAMD_RED_MIN: return run_backward<kMin>(__func__, x, y, index, mean, g, dx, outer, len, inner, ddof, s);
        case CTAMD_RED_VAR: return run_backward<kVar>(__func__, x, y, index, mean, g, dx, outer, len, inner, ddof, s);
        default: return run_backward<kStd>(__func__, x, y, index, mean, g, dx, outer, len, inner, ddof, s);
    }
}

int ctamd_broadcast_reduce_f32(const float* g, const size_t* g_shape, const size_t* t_shape, int rank, float* out, void* stream) {
    if (rank < 0 || rank > kMaxDims) return fail(CTAMD_ERANGE, "%s: at most %d dimensions", __func__, kMaxDims);
    if (rank && (!g_shape || !t_shape)) return fail(CTAMD_EINVAL, "%s: null shape", __func__);
    BroadcastPlan p;
    p.rank = rank;
    p.reduced = 1;
    size_t out_count = 1, g_count = 1, stride = 1;
    for (int d = rank - 1; d >= 0; --d) {
        const size_t ge = g_shape[d], te = t_shape[d];
        if (ge != te && ge != 1 && te != 1) return fail(CTAMD_EINVAL, "%s: extents %zu and %zu do not broadcast", __func__, ge, te);
        p.out_extent[d] = te;
        p.keep_stride[d] = (ge == te && ge != 1) ? stride : 0;
        const bool summed = te == 1 && ge > 1;
        p.red_extent[d] = summed ? ge : 1;
        p.red_stride[d] = summed ? stride : 0;
        if (summed) p.reduced *= ge;
        out_count *= te;
        g_count *= ge;
        stride *= ge;
    }
    for (int d = rank; d < kMaxDims; ++d) p.out_extent[d] = p.red_extent[d] = 1, p.keep_stride[d] = p.red_stride[d] = 0;
    if (out_count == 0) return CTAMD_OK;
    if (!out) return fail(CTAMD_EINVAL, "%s: null output", __func__);
    if (g_count == 0) return ctamd_fill_f32(out, 0.0f, out_count, stream);
    if (!g) return fail(CTAMD_EINVAL, "%s: null input", __func__);
    const size_t blocks = (out_count + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: too many elements", __func__);
    hipLaunchKernelGGL(broadcast_reduce_kernel, dim3(unsigned(blocks)), dim3(kThreads), 0, as_stream(stream), g, out, out_count, p);
    account(4.0 * double(g_count) + 4.0 * double(out_count), double(out_count) * double(p.reduced));
    return launched(__func__);
}

int ctamd_fold_mod_f32(const float* g, float* out, size_t g_count, size_t out_count, void* stream) {
    if (out_count == 0) return CTAMD_OK;
    if (!out || (g_count && !g)) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    const size_t blocks = (out_count + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: too many elements", __func__);
    hipLaunchKernelGGL(fold_mod_kernel, dim3(unsigned(blocks)), dim3(kThreads), 0, as_stream(stream), g, out, g_count, out_count);
    account(4.0 * double(g_count) + 4.0 * double(out_count), double(g_count));
    return launched(__func__);
}

}  // extern "C"
