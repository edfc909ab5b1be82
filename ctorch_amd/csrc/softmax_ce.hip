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

// Barrier for exchanges through LDS only.  __syncthreads() also waits for every outstanding global
// load of the wave (its fence covers global memory), which would make the prefetched next row land
// before the current row is processed - exactly the latency the prefetch is there to hide.  Here
// only LDS traffic (lgkmcnt) is drained before the barrier.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Block-wide reductions whose result every thread receives.  `slot` is LDS of THREADS/64 + 1
// entries; consecutive calls must use distinct slots or be separated by the caller's barrier -
// each call ends with the barrier that makes its slot reusable two calls later.
template <int THREADS, class V, class Fold>
__device__ __forceinline__ V block_all(V v, V* slot, Fold fold) {
    if (THREADS == 64) return v;
    constexpr int W = THREADS / 64;
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    lds_barrier();
    V t = slot[0];
#pragma unroll
    for (int w = 1; w < W; ++w) t = fold(t, slot[w]);
    lds_barrier();
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
    // Rows that need a 1024-thread block (more than 8192 columns) belong to tensors that pass through
    // once and do not fit the caches: their accesses carry the non-temporal hint (one-pass cross
    // entropy 384 -> 358 us, softmax gradient 600 -> 536 us at [8192 x 32000]).  Short rows - the
    // logits of a small classifier - stay plain, so that the next kernel finds them cached.
    static constexpr bool kStream = THREADS == 1024;
    // Branch-free: a group past the end of the row is fetched from a constant pad vector instead
    // (the select is on the address, not on the data), so the loads form one straight-line burst
    // whose results nothing touches until the row is processed - the compiler can then count them
    // exactly when it places its waits, and the next row's loads stay in flight meanwhile.
    __device__ __forceinline__ void load(const float* __restrict__ p, unsigned cols, const float* __restrict__ pad) {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const unsigned e = (threadIdx.x + unsigned(k) * THREADS) * W;
            const float* src = (e < cols) ? p + e : pad;
            if (W == 4) {
                v4f t = kStream ? __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src)) : *reinterpret_cast<const v4f*>(src);
#pragma unroll
                for (int i = 0; i < W; ++i) v[k][i] = t[i];
            } else {
                v[k][0] = *src;
            }
        }
    }
    __device__ __forceinline__ void store(float* __restrict__ p, unsigned cols) const {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const unsigned e = (threadIdx.x + unsigned(k) * THREADS) * W;
            if (e < cols) {
                if (W == 4) {
                    v4f t;
#pragma unroll
                    for (int i = 0; i < W; ++i) t[i] = v[k][i];
                    if (kStream) __builtin_nontemporal_store(t, reinterpret_cast<v4f*>(p + e));
                    else *reinterpret_cast<v4f*>(p + e) = t;
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
            for (int i = 0; i < W; ++i) m = __builtin_fmaxf(m, v[k][i]);
        return m;
    }
    // v <- exp(v - m) (padding lanes hold -inf and give exactly 0); returns this thread's sum
    __device__ __forceinline__ float exp_shifted(float m, const uint64_t* exp2) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
#pragma unroll
            for (int i = 0; i < W; ++i) {
                v[k][i] = cta_expf_nonpos(v[k][i] - m, exp2);
                s += v[k][i];
            }
        return s;
    }
    // sum of exp(v - m) with the bit-exact exponential, v unchanged
    __device__ __forceinline__ float sum_exp(float m, const uint64_t* exp2) const {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
#pragma unroll
            for (int i = 0; i < W; ++i) s += cta_expf_nonpos(v[k][i] - m, exp2);
        return s;
    }
    // v <- exp(v - m) in single precision, within 2 ulp of expf (the hardware exp2 with the lost
    // part of its argument put back)
    __device__ __forceinline__ float exp_shifted_fast(float m) {
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
#pragma unroll
            for (int i = 0; i < W; ++i) {
                v[k][i] = cta_exp_hw_nonpos(v[k][i] - m);
                if ((k * W + i) & 1) s1 += v[k][i]; else s0 += v[k][i];
            }
        return s0 + s1;
    }
    // sum of exp(v - m) without changing v, with the hardware exp2: the loss only needs this sum
    // to ~1e-7 relative (the reference's own sequential sum is no closer), so the forward loss
    // kernels skip the bit-exact exp for it and stay bandwidth-bound
    __device__ __forceinline__ float sum_exp_fast(float m) const {
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
#pragma unroll
            for (int i = 0; i < W; ++i) {
                float e = __builtin_amdgcn_exp2f((v[k][i] - m) * 1.44269504088896340736f);
                if ((k * W + i) & 1) s1 += e; else s0 += e;
            }
        return s0 + s1;
    }
    __device__ __forceinline__ unsigned index(int k, int i) const {
        return (threadIdx.x + unsigned(k) * THREADS) * W + i;
    }
    // group k of another row-shaped operand, fetched when it is needed (keeps register pressure low)
    __device__ __forceinline__ void group(const float* __restrict__ p, unsigned cols, int k, float pad, float (&g)[W]) const {
        const unsigned e = (threadIdx.x + unsigned(k) * THREADS) * W;
        if (e < cols) {
            if (W == 4) {
                v4f t = *reinterpret_cast<const v4f*>(p + e);
#pragma unroll
                for (int i = 0; i < W; ++i) g[i] = t[i];
            } else {
                g[0] = p[e];
            }
        } else {
#pragma unroll
            for (int i = 0; i < W; ++i) g[i] = pad;
        }
    }
};

// The ...Fast variants of the modes that write exp(x - max) / sum (or a function of it) evaluate the
// exponential in single precision (<= 2 ulp) and multiply by 1 / sum; the plain ones return glibc's
// expf bit for bit and the exactly rounded quotient.  kLogSoftmaxFast only forms its row SUM with the
// hardware exponential (its output needs no exponential).
enum Mode { kSoftmax, kCeOnehot, kCeIndex, kCeBwdOnehot, kCeBwdIndex, kSoftmaxBwd, kCeIndexBoth, kCeIndexBothFast,
            kLogSoftmax, kLogSoftmaxFast, kLogSoftmaxBwd, kSoftmaxFast, kCeBwdOnehotFast, kCeBwdIndexFast, kLogSoftmaxBwdFast };
constexpr bool fast_out(int mode) {
    return mode == kSoftmaxFast || mode == kCeBwdOnehotFast || mode == kCeBwdIndexFast || mode == kCeIndexBothFast || mode == kLogSoftmaxBwdFast;
}
constexpr int base_mode(int mode) {
    return mode == kSoftmaxFast ? kSoftmax : mode == kCeBwdOnehotFast ? kCeBwdOnehot : mode == kCeBwdIndexFast ? kCeBwdIndex
         : mode == kCeIndexBothFast ? kCeIndexBoth : mode == kLogSoftmaxBwdFast ? kLogSoftmaxBwd : mode;
}

struct Args {
    const float* x;      // logits / softmax output y (kSoftmaxBwd)
    const float* t;      // one-hot targets / class indices / upstream gradient (kSoftmaxBwd)
    const float* g1;     // 0-D upstream gradient of the loss (backward modes)
    float* out;          // y / dx
    double* partials;    // per-block loss partials (forward loss modes)
    int32_t* status;     // bad-index flag (kCeIndex), may be null
    float* stats;        // kCeIndex: per-row (max, sum of exp(x - max)) for a later backward, may be null
    size_t rows, cols;
    // what a row's register copy holds beyond the row's end: four floats of -inf for logits (exp
    // gives exactly 0) and of 0 for the factors of a dot product, in device memory
    const float* pad_neg_inf;
    const float* pad_zero;
};

// A block walks rows blockIdx.x, blockIdx.x + gridDim.x, ...  For the one-operand modes (softmax,
// class-index cross entropy forward / backward) the next row's loads are issued before the current
// row is processed, so HBM latency hides behind the exp / divide work of the row in hand: with
// 1024-thread blocks only one block fits a CU, and without this the CU would alternate between
// waiting for memory and computing.
template <int MODE_, int THREADS, int ITEMS, int W>
__global__ __launch_bounds__(THREADS) void row_kernel(Args a) {
    constexpr int MODE = base_mode(MODE_);          // what the kernel does
    constexpr bool kFastOut = fast_out(MODE_);      // how it evaluates exp(x - max) / sum
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_f[2][THREADS / 64 + 1];
    __shared__ double s_d[THREADS / 64 + 1];
    stage_exp_table(s_exp2);
    constexpr bool kBoth = (MODE == kCeIndexBoth);
    constexpr bool kLogSm = (MODE == kLogSoftmax || MODE == kLogSoftmaxFast);
    // (a row of 16 groups per thread fills the registers by itself: no second copy to prefetch into)
    constexpr bool kPipelined = (MODE == kSoftmax || MODE == kCeIndex || MODE == kCeBwdIndex || kBoth || kLogSm) && ITEMS <= 8;
    double block_loss = 0.0;
    bool block_bad = false;   // a class index out of range was met (thread 0's copy counts)

    // everything that happens to one row once it sits in `r`; `mloc` is this thread's maximum
    auto process = [&](Row<THREADS, ITEMS, W>& r, size_t row, float mloc) {
        const float m = block_max<THREADS>(mloc, s_f[0]);
        constexpr bool kLossOnly = (MODE == kCeOnehot || MODE == kCeIndex);
        if (kLogSm) {
            // y = (x - m) - log(sum exp(x - m)); rows of 2048 columns or more form the sum with the
            // hardware exponential (~1e-7 relative, i.e. ~1e-7 absolute in its logarithm)
            const float s = block_sum<THREADS>(MODE == kLogSoftmaxFast ? r.sum_exp_fast(m) : r.sum_exp(m, s_exp2), s_f[1]);
            const float lg = cta_logf(s, cta_log_tab);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    const float d = r.v[k][i] - m;
                    r.v[k][i] = d - lg;
                }
            r.store(a.out + row * a.cols, unsigned(a.cols));
            return;
        }
        // loss kernels keep x in r and only need the row sum; the others turn r into exp(x - m)
        const float s = block_sum<THREADS>(kLossOnly ? r.sum_exp_fast(m) : kFastOut ? r.exp_shifted_fast(m) : r.exp_shifted(m, s_exp2), s_f[1]);
        const double rcp_s = 1.0 / double(s);     // e / s below is the exact fp32 quotient (cta_div_rcp)
        const float rcp_sf = 1.0f / s;            // fast output: e * (1 / s)
        if (MODE == kSoftmax) {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) r.v[k][i] = kFastOut ? r.v[k][i] * rcp_sf : cta_div_rcp(r.v[k][i], rcp_s);
            r.store(a.out + row * a.cols, unsigned(a.cols));
        } else if (MODE == kCeOnehot) {
            // -sum_j t_j * log(max(e_j / s, 1e-10)); terms with t_j == 0 contribute exactly 0
            Row<THREADS, ITEMS, W> q;
            q.load(a.t + row * a.cols, unsigned(a.cols), a.pad_zero);
            double loss = 0.0;
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    float tj = q.v[k][i];
                    if (tj != 0.0f) {
                        float p = cta_div_rcp(cta_expf_nonpos(r.v[k][i] - m, s_exp2), rcp_s);
                        p = (p < 1e-10f) ? 1e-10f : p;
                        float lg = float(log(double(p)));
                        loss -= double(tj * lg);
                    }
                }
            loss = block_sum<THREADS>(loss, s_d);
            block_loss += loss;
        } else if (MODE == kCeIndex) {
            const int c = class_index(a.t[row]);
            if (threadIdx.x == 0 && a.stats) {
                a.stats[2 * row] = m;
                a.stats[2 * row + 1] = s;
            }
            if (c < 0 || c >= int(a.cols)) {
                block_bad = true;
                block_loss += double(__builtin_nanf(""));
            } else {
                // the thread that holds column c publishes exp(x_c - m): pick x_c by selects, then
                // one exact exp per thread (not one per element)
                float xc = 0.0f;
                bool mine = false;
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                    for (int i = 0; i < W; ++i) {
                        const bool hit = r.index(k, i) == unsigned(c);
                        xc = hit ? r.v[k][i] : xc;
                        mine = mine || hit;
                    }
                float ec = mine ? cta_expf_nonpos(xc - m, s_exp2) : 0.0f;
                ec = block_sum<THREADS>(ec, s_f[0]);
                float p = ec / s;
                p = (p < 1e-10f) ? 1e-10f : p;
                block_loss -= double(float(log(double(p))));
            }
        } else if (kBoth) {
            // loss and gradient from one visit of the row: r holds e = exp(x - m), s is its sum;
            // the gradient is the one for an upstream gradient of 1 (d * 1.0f is d)
            // (the class index is read here, not earlier: a wait for it right after the next row's
            // loads were issued would wait for those as well)
            const int c = class_index(a.t[row]);
            const bool ok = c >= 0 && c < int(a.cols);
            // which of this thread's elements is column c, as one number (k * W + i, or -1): comparing
            // it with each element's constant position keeps 32 column indices out of the registers
            const int q = (ok ? c / W : -1) - int(threadIdx.x);
            const int slot = (q >= 0 && q % THREADS == 0) ? (q / THREADS) * W + c % W : -1;
            // exp(x_c - m) once more from the logit itself, by every thread (row and c are uniform:
            // one broadcast read of a line the row's loads have just brought in) - the same value as
            // the row's own element, with no search through the registers and no exchange
            const float xc = ok ? a.x[row * a.cols + size_t(c)] : 0.0f;
            const float ec = kFastOut ? cta_exp_hw_nonpos(xc - m) : cta_expf_nonpos(xc - m, s_exp2);
            if (!ok) {
                block_bad = true;
                block_loss += double(__builtin_nanf(""));
            } else {
                float p = ec / s;
                p = (p < 1e-10f) ? 1e-10f : p;
                block_loss -= double(float(log(double(p))));
            }
            // the class column's gradient 0 + (e_c / s - 1); every other element 0 + (e / s - 0) = e / s
            const float smc = kFastOut ? ec * rcp_sf : cta_div_rcp(ec, rcp_s);
            const float dc = 0.0f + (smc - 1.0f);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    const float sm = kFastOut ? r.v[k][i] * rcp_sf : cta_div_rcp(r.v[k][i], rcp_s);
                    r.v[k][i] = (slot == k * W + i) ? dc : sm;
                }
            r.store(a.out + row * a.cols, unsigned(a.cols));
        } else {   // kCeBwdOnehot / kCeBwdIndex: dx = 0 + (e / s - t) * g (the tape adds it to a zero-filled buffer)
            const float g = a.g1[0];
            if (MODE == kCeBwdOnehot) {
#pragma unroll
                for (int k = 0; k < ITEMS; ++k) {
                    float tq[W];
                    r.group(a.t + row * a.cols, unsigned(a.cols), k, 0.0f, tq);
#pragma unroll
                    for (int i = 0; i < W; ++i) {
                        float sm = kFastOut ? r.v[k][i] * rcp_sf : cta_div_rcp(r.v[k][i], rcp_s);
                        float d = sm - tq[i];
                        r.v[k][i] = 0.0f + d * g;
                    }
                }
            } else {
                const int c = class_index(a.t[row]);
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                    for (int i = 0; i < W; ++i) {
                        float sm = kFastOut ? r.v[k][i] * rcp_sf : cta_div_rcp(r.v[k][i], rcp_s);
                        float d = sm - ((r.index(k, i) == unsigned(c)) ? 1.0f : 0.0f);
                        r.v[k][i] = 0.0f + d * g;
                    }
            }
            r.store(a.out + row * a.cols, unsigned(a.cols));
        }
    };

    const size_t stride = gridDim.x;
    size_t row = blockIdx.x;
    if (MODE == kLogSoftmaxBwd) {
        for (; row < a.rows; row += stride) {
            // r = y = log_softmax(x), q = g: d = sum g, dx = g - exp(y) * d
            Row<THREADS, ITEMS, W> r, q;
            r.load(a.x + row * a.cols, unsigned(a.cols), a.pad_neg_inf);
            q.load(a.t + row * a.cols, unsigned(a.cols), a.pad_zero);
            float d = 0.0f;
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) d += q.v[k][i];
            d = block_sum<THREADS>(d, s_f[0]);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    const float t = (kFastOut ? cta_exp_hw(r.v[k][i]) : cta_expf_tab(r.v[k][i], s_exp2)) * d;
                    r.v[k][i] = q.v[k][i] - t;
                }
            r.store(a.out + row * a.cols, unsigned(a.cols));
        }
    } else if (MODE == kSoftmaxBwd) {
        for (; row < a.rows; row += stride) {
            // r = y, q = g: d = sum g*y, dx = y * (g - d)
            Row<THREADS, ITEMS, W> r, q;
            r.load(a.x + row * a.cols, unsigned(a.cols), a.pad_zero);
            q.load(a.t + row * a.cols, unsigned(a.cols), a.pad_zero);
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
            r.store(a.out + row * a.cols, unsigned(a.cols));
        }
    } else if (kPipelined) {
        // Two register copies of a row, alternating.  Per row: take the thread's maximum (the first
        // touch of the row's data, i.e. the wait for its loads), THEN issue the next row's loads,
        // then do the exp / divide / store work, during which those loads are in flight.  The
        // order matters: loads and stores share one in-order counter on this architecture, and a
        // wait with both kinds outstanding drains everything - issued before the first touch, the
        // new loads would be waited for at once.
        Row<THREADS, ITEMS, W> ra, rb;
        if (row < a.rows) ra.load(a.x + row * a.cols, unsigned(a.cols), a.pad_neg_inf);
        while (row < a.rows) {
            float mloc = ra.max();
            asm volatile("" : "+v"(mloc) : : "memory");   // the loads below may not move above this
            if (row + stride < a.rows) rb.load(a.x + (row + stride) * a.cols, unsigned(a.cols), a.pad_neg_inf);
            __builtin_amdgcn_sched_barrier(0);
            process(ra, row, mloc);
            row += stride;
            if (row >= a.rows) break;
            mloc = rb.max();
            asm volatile("" : "+v"(mloc) : : "memory");
            if (row + stride < a.rows) ra.load(a.x + (row + stride) * a.cols, unsigned(a.cols), a.pad_neg_inf);
            __builtin_amdgcn_sched_barrier(0);
            process(rb, row, mloc);
            row += stride;
        }
    } else {
        for (; row < a.rows; row += stride) {
            Row<THREADS, ITEMS, W> r;
            r.load(a.x + row * a.cols, unsigned(a.cols), a.pad_neg_inf);
            process(r, row, r.max());
        }
    }
    if ((MODE == kCeOnehot || MODE == kCeIndex || kBoth) && threadIdx.x == 0) {
        a.partials[blockIdx.x] = block_loss;
        if ((MODE == kCeIndex || kBoth) && a.status) a.partials[gridDim.x + blockIdx.x] = block_bad ? 1.0 : 0.0;
    }
}

// Streaming variant for rows that do not fit a block's registers: pass 1 keeps an online
// (max, sum) pair per thread - sum is rescaled by exp(old_max - new_max) whenever the max grows -
// pass 2 re-reads the row.  The rescaled sum differs from sum(exp(x - max)) by rounding only.
// The same for softmax and its gradient with 128-bit accesses (rows of a multiple of four columns,
// 16-byte aligned): four vectors in flight per thread, the row sum of the first sweep from the
// hardware exp2 (only the sum is formed from it, ~1e-7 relative; the output sweep uses the bit-exact
// exponential and the exact quotient), plain loads so that the second sweep finds the row in the
// memory-side cache (one block per CU keeps 256 rows in flight), results written past the caches.
template <int MODE_>
__global__ __launch_bounds__(1024) void row_stream_vec_kernel(Args a) {
    constexpr int THREADS = 1024, U = 4;
    constexpr int MODE = base_mode(MODE_);
    constexpr bool kFastOut = fast_out(MODE_);
    static_assert(MODE == kSoftmax || MODE == kSoftmaxBwd || MODE == kLogSoftmaxFast || MODE == kLogSoftmaxBwd,
                  "only the modes that write a row-shaped result");
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_f[2][THREADS / 64 + 1];
    stage_exp_table(s_exp2);
    const unsigned n4 = unsigned(a.cols >> 2);
    for (size_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const v4f* __restrict__ xr = reinterpret_cast<const v4f*>(a.x + row * a.cols);
        v4f* __restrict__ outr = reinterpret_cast<v4f*>(a.out + row * a.cols);
        if (MODE == kLogSoftmaxBwd) {
            // d = sum g (first sweep over g alone), dx = g - exp(y) * d
            const v4f* __restrict__ gr = reinterpret_cast<const v4f*>(a.t + row * a.cols);
            float d0 = 0.0f, d1 = 0.0f;
            unsigned i = threadIdx.x;
            for (; i + (U - 1) * THREADS < n4; i += U * THREADS) {
                v4f g[U];
#pragma unroll
                for (int u = 0; u < U; ++u) g[u] = gr[i + u * THREADS];
#pragma unroll
                for (int u = 0; u < U; ++u) { d0 += g[u][0] + g[u][1]; d1 += g[u][2] + g[u][3]; }
            }
            for (; i < n4; i += THREADS) { const v4f g = gr[i]; d0 += g[0] + g[1]; d1 += g[2] + g[3]; }
            const float d = block_sum<THREADS>(d0 + d1, s_f[0]);
            auto give = [&](const v4f& y, const v4f& g, unsigned at) {
                v4f o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float t = (kFastOut ? cta_exp_hw(y[e]) : cta_expf_tab(y[e], s_exp2)) * d;
                    o[e] = g[e] - t;
                }
                __builtin_nontemporal_store(o, outr + at);
            };
            i = threadIdx.x;
            for (; i + (U / 2 - 1) * THREADS < n4; i += (U / 2) * THREADS) {
                v4f y[U / 2], g[U / 2];
#pragma unroll
                for (int u = 0; u < U / 2; ++u) { y[u] = xr[i + u * THREADS]; g[u] = gr[i + u * THREADS]; }
#pragma unroll
                for (int u = 0; u < U / 2; ++u) give(y[u], g[u], i + u * THREADS);
            }
            for (; i < n4; i += THREADS) give(xr[i], gr[i], i);
            continue;
        }
        if (MODE == kSoftmaxBwd) {
            const v4f* __restrict__ gr = reinterpret_cast<const v4f*>(a.t + row * a.cols);
            float d0 = 0.0f, d1 = 0.0f;
            unsigned i = threadIdx.x;
            for (; i + (U / 2 - 1) * THREADS < n4; i += (U / 2) * THREADS) {
                v4f y[U / 2], g[U / 2];
#pragma unroll
                for (int u = 0; u < U / 2; ++u) { y[u] = xr[i + u * THREADS]; g[u] = gr[i + u * THREADS]; }
#pragma unroll
                for (int u = 0; u < U / 2; ++u) {
                    d0 += g[u][0] * y[u][0] + g[u][1] * y[u][1];
                    d1 += g[u][2] * y[u][2] + g[u][3] * y[u][3];
                }
            }
            for (; i < n4; i += THREADS) {
                const v4f y = xr[i], g = gr[i];
                d0 += g[0] * y[0] + g[1] * y[1];
                d1 += g[2] * y[2] + g[3] * y[3];
            }
            const float d = block_sum<THREADS>(d0 + d1, s_f[0]);
            i = threadIdx.x;
            for (; i + (U / 2 - 1) * THREADS < n4; i += (U / 2) * THREADS) {
                v4f y[U / 2], g[U / 2];
#pragma unroll
                for (int u = 0; u < U / 2; ++u) { y[u] = xr[i + u * THREADS]; g[u] = gr[i + u * THREADS]; }
#pragma unroll
                for (int u = 0; u < U / 2; ++u) {
                    v4f o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = y[u][e] * (g[u][e] - d);
                    __builtin_nontemporal_store(o, outr + i + u * THREADS);
                }
            }
            for (; i < n4; i += THREADS) {
                const v4f y = xr[i], g = gr[i];
                v4f o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = y[e] * (g[e] - d);
                __builtin_nontemporal_store(o, outr + i);
            }
            continue;
        }
        float m = kNegInf, s = 0.0f;
        auto take = [&](const v4f& v) {
            const float vm = __builtin_fmaxf(__builtin_fmaxf(v[0], v[1]), __builtin_fmaxf(v[2], v[3]));
            if (vm > m) {
                s *= __builtin_amdgcn_exp2f((m - vm) * 1.44269504088896340736f);      // exp2(-inf) = 0 at the first vector
                m = vm;
            }
            const float b = (m == kNegInf) ? 0.0f : m;
            s += (__builtin_amdgcn_exp2f((v[0] - b) * 1.44269504088896340736f) + __builtin_amdgcn_exp2f((v[1] - b) * 1.44269504088896340736f)) +
                 (__builtin_amdgcn_exp2f((v[2] - b) * 1.44269504088896340736f) + __builtin_amdgcn_exp2f((v[3] - b) * 1.44269504088896340736f));
        };
        unsigned i = threadIdx.x;
        for (; i + (U - 1) * THREADS < n4; i += U * THREADS) {
            v4f v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = xr[i + u * THREADS];
#pragma unroll
            for (int u = 0; u < U; ++u) take(v[u]);
        }
        for (; i < n4; i += THREADS) take(xr[i]);
        const float M = block_max<THREADS>(m, s_f[0]);
        s = (m == kNegInf) ? 0.0f : s * __builtin_amdgcn_exp2f((m - M) * 1.44269504088896340736f);
        const float S = block_sum<THREADS>(s, s_f[1]);
        const double rcp = 1.0 / double(S);
        const float rcp_f = 1.0f / S;
        const float lg = (MODE == kLogSoftmaxFast) ? cta_logf(S, cta_log_tab) : 0.0f;
        auto give = [&](const v4f& v, unsigned at) {
            v4f o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (MODE == kLogSoftmaxFast) {
                    const float d = v[e] - M;
                    o[e] = d - lg;
                } else if (kFastOut) {
                    o[e] = cta_exp_hw_nonpos(v[e] - M) * rcp_f;
                } else {
                    o[e] = cta_div_rcp(cta_expf_nonpos(v[e] - M, s_exp2), rcp);
                }
            }
            __builtin_nontemporal_store(o, outr + at);
        };
        i = threadIdx.x;
        for (; i + (U - 1) * THREADS < n4; i += U * THREADS) {
            v4f v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = xr[i + u * THREADS];
#pragma unroll
            for (int u = 0; u < U; ++u) give(v[u], i + u * THREADS);
        }
        for (; i < n4; i += THREADS) give(xr[i], i);
    }
}

// Rows of more than 32768 and at most 65536 columns (128-bit accesses): the two sweeps of the kernel
// above with the operand that both sweeps need kept on the chip between them - sixteen 128-bit words
// per thread, eight in registers and eight in LDS (128 KiB per block; one block of 1024 threads per CU)
// - so that it is read from memory once:
//   softmax, log-softmax        x kept:  8 B/elem moved instead of 12
//   softmax gradient            y kept: 16 instead of 20 (g, which the first sweep needs for the row's
//                                       dot product and the second for the result, is read twice)
//   log-softmax gradient        g kept: 12 instead of 16
// The arithmetic, and so every bit of the results, is the kernel's above.
constexpr int kKeepRegs = 8, kKeepLds = 8;
constexpr unsigned kKeepVectors = (kKeepRegs + kKeepLds) * 1024;
template <int MODE_>
__global__ __launch_bounds__(1024) void row_keep_kernel(Args a) {
    constexpr int THREADS = 1024;
    constexpr int MODE = base_mode(MODE_);
    constexpr bool kFastOut = fast_out(MODE_);
    static_assert(MODE == kSoftmax || MODE == kSoftmaxBwd || MODE == kLogSoftmaxFast || MODE == kLogSoftmaxBwd,
                  "only the modes that write a row-shaped result");
    static_assert(kKeepRegs % 2 == 0 && kKeepLds % 2 == 0, "words are taken two at a time");
    extern __shared__ v4f s_keep[];                 // [kKeepLds][THREADS]
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_f[2][THREADS / 64 + 1];
    stage_exp_table(s_exp2);
    const unsigned n4 = unsigned(a.cols >> 2);      // at most kKeepVectors
    const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
    v4f* const mine = s_keep + threadIdx.x;
    for (size_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const v4f* __restrict__ xr = reinterpret_cast<const v4f*>(a.x + row * a.cols);
        const v4f* __restrict__ gr = reinterpret_cast<const v4f*>(a.t + row * a.cols);
        v4f* __restrict__ outr = reinterpret_cast<v4f*>(a.out + row * a.cols);
        v4f keep[kKeepRegs];
        // A sweep visits the row's words two at a time: first the words kept in registers (unrolled:
        // their register numbers must be constants), then - in a loop - the words kept in LDS.
        // `first(i0, i1, ok0, ok1, slot0, slot1)` is handed two word indices, whether they lie inside the
        // row, and where the kept copies live.
        auto sweep = [&](auto&& visit) {
#pragma unroll
            for (int u = 0; u < kKeepRegs; u += 2) {
                const unsigned i0 = threadIdx.x + unsigned(u) * THREADS, i1 = i0 + THREADS;
                visit(i0, i1, i0 < n4, i1 < n4, keep[u], keep[u + 1]);
                __builtin_amdgcn_sched_barrier(0);          // the next pair's loads stay behind this pair's work
            }
#pragma unroll 1
            for (int u = 0; u < kKeepLds; u += 2) {
                const unsigned i0 = threadIdx.x + unsigned(kKeepRegs + u) * THREADS, i1 = i0 + THREADS;
                if (i0 >= n4) break;
                visit(i0, i1, true, i1 < n4, mine[u * THREADS], mine[(u + 1) * THREADS]);
            }
        };
        if (MODE == kSoftmaxBwd) {
            // d = sum g * y with y left on the chip; then dx = y * (g - d) from the kept y and g read again
            float d0 = 0.0f, d1 = 0.0f;
            sweep([&](unsigned i0, unsigned i1, bool ok0, bool ok1, v4f& k0, v4f& k1) {
                const v4f y0 = ok0 ? xr[i0] : zero, y1 = ok1 ? xr[i1] : zero;
                const v4f g0 = ok0 ? gr[i0] : zero, g1 = ok1 ? gr[i1] : zero;
                d0 += g0[0] * y0[0] + g0[1] * y0[1];
                d1 += g0[2] * y0[2] + g0[3] * y0[3];
                d0 += g1[0] * y1[0] + g1[1] * y1[1];
                d1 += g1[2] * y1[2] + g1[3] * y1[3];
                k0 = y0;
                k1 = y1;
            });
            const float d = block_sum<THREADS>(d0 + d1, s_f[0]);
            sweep([&](unsigned i0, unsigned i1, bool ok0, bool ok1, v4f& k0, v4f& k1) {
                const v4f g0 = ok0 ? __builtin_nontemporal_load(gr + i0) : zero, g1 = ok1 ? __builtin_nontemporal_load(gr + i1) : zero;
                v4f o0, o1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o0[e] = k0[e] * (g0[e] - d);
                    o1[e] = k1[e] * (g1[e] - d);
                }
                if (ok0) __builtin_nontemporal_store(o0, outr + i0);
                if (ok1) __builtin_nontemporal_store(o1, outr + i1);
            });
            continue;
        }
        if (MODE == kLogSoftmaxBwd) {
            // d = sum g with g left on the chip; then dx = g - exp(y) * d from the kept g and y read once
            float d0 = 0.0f, d1 = 0.0f;
            sweep([&](unsigned i0, unsigned i1, bool ok0, bool ok1, v4f& k0, v4f& k1) {
                k0 = ok0 ? __builtin_nontemporal_load(gr + i0) : zero;
                k1 = ok1 ? __builtin_nontemporal_load(gr + i1) : zero;
                d0 += (k0[0] + k0[1]) + (k1[0] + k1[1]);
                d1 += (k0[2] + k0[3]) + (k1[2] + k1[3]);
            });
            const float d = block_sum<THREADS>(d0 + d1, s_f[0]);
            sweep([&](unsigned i0, unsigned i1, bool ok0, bool ok1, v4f& k0, v4f& k1) {
                const v4f y0 = ok0 ? __builtin_nontemporal_load(xr + i0) : zero, y1 = ok1 ? __builtin_nontemporal_load(xr + i1) : zero;
                v4f o0, o1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o0[e] = k0[e] - (kFastOut ? cta_exp_hw(y0[e]) : cta_expf_tab(y0[e], s_exp2)) * d;
                    o1[e] = k1[e] - (kFastOut ? cta_exp_hw(y1[e]) : cta_expf_tab(y1[e], s_exp2)) * d;
                }
                if (ok0) __builtin_nontemporal_store(o0, outr + i0);
                if (ok1) __builtin_nontemporal_store(o1, outr + i1);
            });
            continue;
        }
        // softmax / log-softmax: the online (max, sum) pair of the kernel above over the words as they
        // arrive, x left on the chip; then the result from the kept x
        float m = kNegInf, s = 0.0f;
        auto take = [&](const v4f& v) {
            const float vm = __builtin_fmaxf(__builtin_fmaxf(v[0], v[1]), __builtin_fmaxf(v[2], v[3]));
            if (vm > m) {
                s *= __builtin_amdgcn_exp2f((m - vm) * 1.44269504088896340736f);
                m = vm;
            }
            const float b = (m == kNegInf) ? 0.0f : m;
            s += (__builtin_amdgcn_exp2f((v[0] - b) * 1.44269504088896340736f) + __builtin_amdgcn_exp2f((v[1] - b) * 1.44269504088896340736f)) +
                 (__builtin_amdgcn_exp2f((v[2] - b) * 1.44269504088896340736f) + __builtin_amdgcn_exp2f((v[3] - b) * 1.44269504088896340736f));
        };
        sweep([&](unsigned i0, unsigned i1, bool ok0, bool ok1, v4f& k0, v4f& k1) {
            k0 = ok0 ? __builtin_nontemporal_load(xr + i0) : zero;
            k1 = ok1 ? __builtin_nontemporal_load(xr + i1) : zero;
            if (ok0) take(k0);
            if (ok1) take(k1);
        });
        const float M = block_max<THREADS>(m, s_f[0]);
        s = (m == kNegInf) ? 0.0f : s * __builtin_amdgcn_exp2f((m - M) * 1.44269504088896340736f);
        const float S = block_sum<THREADS>(s, s_f[1]);
        const double rcp = 1.0 / double(S);
        const float rcp_f = 1.0f / S;
        const float lg = (MODE == kLogSoftmaxFast) ? cta_logf(S, cta_log_tab) : 0.0f;
        auto result = [&](const v4f& v) {
            v4f o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (MODE == kLogSoftmaxFast) {
                    const float d = v[e] - M;
                    o[e] = d - lg;
                } else if (kFastOut) {
                    o[e] = cta_exp_hw_nonpos(v[e] - M) * rcp_f;
                } else {
                    o[e] = cta_div_rcp(cta_expf_nonpos(v[e] - M, s_exp2), rcp);
                }
            }
            return o;
        };
        sweep([&](unsigned i0, unsigned i1, bool ok0, bool ok1, v4f& k0, v4f& k1) {
            if (ok0) __builtin_nontemporal_store(result(k0), outr + i0);
            if (ok1) __builtin_nontemporal_store(result(k1), outr + i1);
        });
    }
}

template <int MODE_>
__global__ __launch_bounds__(1024) void row_stream_kernel(Args a) {
    constexpr int THREADS = 1024;
    constexpr int MODE = base_mode(MODE_);          // this path (ragged or unaligned long rows) keeps the exact routines
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_f[2][THREADS / 64 + 1];
    __shared__ double s_d[THREADS / 64 + 1];
    stage_exp_table(s_exp2);
    double block_loss = 0.0;
    bool block_bad = false;   // a class index out of range was met (thread 0's copy counts)
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
        if (MODE == kLogSoftmaxBwd) {
            const float* gr = a.t + row * a.cols;
            float d = 0.0f;
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) d += gr[j];
            d = block_sum<THREADS>(d, s_f[0]);
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) {
                const float t = cta_expf_tab(xr[j], s_exp2) * d;
                a.out[row * a.cols + j] = gr[j] - t;
            }
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
                a.out[row * a.cols + j] = cta_div_rcp(cta_expf_tab(xr[j] - M, s_exp2), 1.0 / double(S));
        } else if (MODE == kLogSoftmax || MODE == kLogSoftmaxFast) {
            const float lg = cta_logf(S, cta_log_tab);
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) {
                const float d = xr[j] - M;
                a.out[row * a.cols + j] = d - lg;
            }
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
            const int c = class_index(a.t[row]);
            if (threadIdx.x == 0 && a.stats) {
                a.stats[2 * row] = M;
                a.stats[2 * row + 1] = S;
            }
            if (c < 0 || c >= int(a.cols)) {
                block_bad = true;
                block_loss += double(__builtin_nanf(""));
            } else {
                float p = cta_expf_tab(xr[c] - M, s_exp2) / S;
                p = (p < 1e-10f) ? 1e-10f : p;
                block_loss -= double(float(log(double(p))));
            }
        } else {
            const float g = a.g1[0];
            const int c = (MODE == kCeBwdIndex) ? class_index(a.t[row]) : -1;
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) {
                float sm = cta_expf_tab(xr[j] - M, s_exp2) / S;
                float tj = (MODE == kCeBwdOnehot) ? a.t[row * a.cols + j] : ((j == size_t(c) && c >= 0) ? 1.0f : 0.0f);
                float d = sm - tj;
                a.out[row * a.cols + j] = 0.0f + d * g;
            }
        }
    }
    if ((MODE == kCeOnehot || MODE == kCeIndex) && threadIdx.x == 0) {
        a.partials[blockIdx.x] = block_loss;
        if (MODE == kCeIndex && a.status) a.partials[gridDim.x + blockIdx.x] = block_bad ? 1.0 : 0.0;
    }
}

// Class-index cross entropy, forward, for long rows: a single pass with an online (max, sum) pair
// per thread.  Nothing of the row is kept, so a 256-thread block per row needs few registers, many
// blocks share a CU and the kernel runs at memory speed (the register-resident variant, one
// 1024-thread block per CU, reached 3.9 TB/s on 8192 x 32000).  Each 128-bit vector first raises
// the running maximum (rescaling the running sum by exp(old - new) when it grows) and then adds its
// four exp(x - max) terms, all with the hardware exp2: only the row's log-sum is needed, to ~1e-7
// relative.  The target logit's own term exp(x_c - max) is evaluated with the bit-exact exp.
constexpr float kLog2e = 1.44269504088896340736f;

template <bool VEC>
__global__ __launch_bounds__(256) void ce_index_online_kernel(Args a) {
    constexpr int THREADS = 256;
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_f[2][THREADS / 64 + 1];
    stage_exp_table(s_exp2);
    double block_loss = 0.0;
    bool block_bad = false;   // a class index out of range was met (thread 0's copy counts)
    for (size_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const float* __restrict__ xr = a.x + row * a.cols;
        float m = kNegInf, s = 0.0f;
        auto absorb4 = [&](v4f v) {
            float cm = __builtin_fmaxf(__builtin_fmaxf(v[0], v[1]), __builtin_fmaxf(v[2], v[3]));
            if (cm > m) {
                s *= __builtin_amdgcn_exp2f((m - cm) * kLog2e);     // exp2(-inf) = 0 on the first vector
                m = cm;
            }
            const float b = (m == kNegInf) ? 0.0f : m;              // all -inf so far: terms are exp(-inf) = 0, not NaN
            s += (__builtin_amdgcn_exp2f((v[0] - b) * kLog2e) + __builtin_amdgcn_exp2f((v[1] - b) * kLog2e)) +
                 (__builtin_amdgcn_exp2f((v[2] - b) * kLog2e) + __builtin_amdgcn_exp2f((v[3] - b) * kLog2e));
        };
        if (VEC) {
            const unsigned n4 = unsigned(a.cols >> 2);
            constexpr int U = 8;
            unsigned i = threadIdx.x;
            for (; i + (U - 1) * THREADS < n4; i += U * THREADS) {
                v4f v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(xr) + i + u * THREADS);
#pragma unroll
                for (int u = 0; u < U; ++u) absorb4(v[u]);
            }
            for (; i < n4; i += THREADS) absorb4(reinterpret_cast<const v4f*>(xr)[i]);
        } else {
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) {
                float v = xr[j];
                if (v > m) {
                    s *= __builtin_amdgcn_exp2f((m - v) * kLog2e);
                    m = v;
                }
                s += __builtin_amdgcn_exp2f((v - ((m == kNegInf) ? 0.0f : m)) * kLog2e);
            }
        }
        const float M = block_max<THREADS>(m, s_f[0]);
        s = (m == kNegInf) ? 0.0f : s * __builtin_amdgcn_exp2f((m - M) * kLog2e);
        const float S = block_sum<THREADS>(s, s_f[1]);
        const int c = class_index(a.t[row]);
        if (threadIdx.x == 0 && a.stats) {
            a.stats[2 * row] = M;
            a.stats[2 * row + 1] = S;
        }
        if (c < 0 || c >= int(a.cols)) {
            block_bad = true;
            block_loss += double(__builtin_nanf(""));
        } else if (threadIdx.x == 0) {
            float p = cta_expf_nonpos(xr[c] - M, s_exp2) / S;
            p = (p < 1e-10f) ? 1e-10f : p;
            block_loss -= double(float(log(double(p))));
        }
    }
    if (threadIdx.x == 0) {
        a.partials[blockIdx.x] = block_loss;
        if (a.status) a.partials[gridDim.x + blockIdx.x] = block_bad ? 1.0 : 0.0;
    }
}

// Class-index cross entropy, backward, from the per-row (max, sum) that the forward pass left
// behind: dx = (exp(x - max) / sum - onehot) * g needs no reduction any more, so it is a pure
// streaming kernel - nothing of the row is kept, few registers, 8 blocks of 256 threads per CU,
// the bit-exact exp and the exact quotient of many rows in flight under each other's loads.
// FAST (rows of 2048 columns or more, whose sum already came from the hardware exponential, ~1e-7
// relative): the same exponential and a multiplication by 1/sum here too, which leaves the kernel
// to the memory stream; the result stays within ~2e-7 * |g| of the exact form.
template <bool VEC, bool FAST>
__global__ __launch_bounds__(256) void ce_bwd_stats_kernel(Args a) {
    constexpr int THREADS = 256;
    __shared__ uint64_t s_exp2[32];
    stage_exp_table(s_exp2);
    const float g = a.g1[0];
    for (size_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const float* __restrict__ xr = a.x + row * a.cols;
        float* __restrict__ outr = a.out + row * a.cols;
        const float M = a.stats[2 * row];
        const double rcp_s = 1.0 / double(a.stats[2 * row + 1]);
        const float rcp_sf = float(rcp_s);
        const unsigned c = unsigned(class_index(a.t[row]));
        auto one = [&](float v, unsigned j) {
            float sm = FAST ? cta_exp_hw_nonpos(v - M) * rcp_sf
                            : cta_div_rcp(cta_expf_nonpos(v - M, s_exp2), rcp_s);
            return 0.0f + (sm - ((j == c) ? 1.0f : 0.0f)) * g;
        };
        if (VEC) {
            const unsigned n4 = unsigned(a.cols >> 2);
            constexpr int U = 4;
            auto finish4 = [&](v4f v, unsigned i4) {
                v4f o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = one(v[e], i4 * 4 + e);
                __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(outr) + i4);
            };
            unsigned i = threadIdx.x;
            for (; i + (U - 1) * THREADS < n4; i += U * THREADS) {
                v4f v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(xr) + i + u * THREADS);
#pragma unroll
                for (int u = 0; u < U; ++u) finish4(v[u], i + u * THREADS);
            }
            for (; i < n4; i += THREADS) finish4(reinterpret_cast<const v4f*>(xr)[i], i);
        } else {
            for (size_t j = threadIdx.x; j < a.cols; j += THREADS) outr[j] = one(xr[j], unsigned(j));
        }
    }
}

// out[0] = float(sum of partials), folded in a fixed order; status[0] (when given) = whether any
// block flagged a bad class index in the second half of the partials (every block writes its flag, so
// nothing has to be cleared beforehand).
__global__ __launch_bounds__(256) void loss_stage2(const double* __restrict__ partials, unsigned count,
                                                   float* __restrict__ out, int32_t* __restrict__ status) {
    __shared__ double s_d[256 / 64 + 1];
    double t = 0.0, bad = 0.0;
    // eight loads (sixteen with the flags) in flight, added in the order of i
    for (unsigned i0 = threadIdx.x; i0 < count; i0 += 256 * 8) {
        double p[8], f[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const unsigned i = i0 + 256u * u;
            p[u] = i < count ? partials[i] : 0.0;
            f[u] = (status && i < count) ? partials[count + i] : 0.0;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (i0 + 256u * u < count) { t += p[u]; bad += f[u]; }
    }
    t = block_sum<256>(t, s_d);
    if (status) {
        __syncthreads();
        bad = block_sum<256>(bad, s_d);
    }
    if (threadIdx.x == 0) {
        out[0] = float(t);
        if (status) status[0] = bad > 0.0 ? 1 : 0;
    }
}

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
    else {
        // rows of 2048 columns or more never reach these two modes (they go to the online forward
        // kernel and to the long-row one-pass kernel): the 1024-thread shapes are not built for them
        // (nor reach them in the exact forms below when the library runs in its fast mode, and vice versa -
        // but both are built: the mode is a run-time switch)
        if constexpr (MODE == kCeIndex || MODE == kCeIndexBoth || MODE == kLogSoftmax) {
            return false;
        } else {
            if (groups <= 1024 * 2) launch_cfg<MODE, 1024, 2, W>(a, grid, s);
            else if constexpr (MODE == kLogSoftmaxBwd) return false;   // two resident rows and the double-precision exponential do not fit 128 registers
            else if (groups <= 1024 * 8) launch_cfg<MODE, 1024, 8, W>(a, grid, s);
            else if constexpr (MODE == kSoftmaxFast && W == 4) {
                // up to 65536 columns: the whole row in registers (64 per thread), one row at a time
                if (groups <= 1024 * 16) launch_cfg<MODE, 1024, 16, W>(a, grid, s);
                else return false;
            } else return false;
        }
    }
    return true;
}

template <int MODE_>
int run_rows(const char* name, Args a, float* loss_out, void* stream) {
    constexpr int MODE = base_mode(MODE_);
    constexpr bool kBoth = (MODE == kCeIndexBoth);
    constexpr bool kLoss = (MODE == kCeOnehot || MODE == kCeIndex || kBoth);
    constexpr bool kIndexLoss = (MODE == kCeIndex || kBoth);
    constexpr bool kWrites = !kLoss || kBoth;                          // a [rows, cols] result
    if (kLoss && !loss_out) return fail(CTAMD_EINVAL, "%s: null output", name);
    hipStream_t s = as_stream(stream);
    if (a.rows == 0 || a.cols == 0) {
        if (kLoss) return ctamd_fill_f32(loss_out, 0.0f, 1, stream);
        return CTAMD_OK;
    }
    constexpr bool kLogSm = (MODE == kLogSoftmax || MODE == kLogSoftmaxFast);
    if (!a.x || (!a.t && MODE != kSoftmax && !kLogSm)) return fail(CTAMD_EINVAL, "%s: null input", name);
    if (kWrites && !a.out) return fail(CTAMD_EINVAL, "%s: null output", name);
    if ((MODE == kCeBwdOnehot || MODE == kCeBwdIndex) && !a.g1) return fail(CTAMD_EINVAL, "%s: null upstream gradient", name);
    if (a.rows > (size_t(1) << 62) / a.cols) return fail(CTAMD_ERANGE, "%s: rows*cols overflows", name);
    if (a.cols > size_t(0x7fffffff)) return fail(CTAMD_ERANGE, "%s: more than 2^31-1 columns", name);
    a.pad_neg_inf = pad_neg_inf();
    a.pad_zero = pad_zero();
    if (!a.pad_zero) return CTAMD_EINVAL;
    {
        // algorithmic bytes per element: logits in (+ one-hot target in) (+ result out); a class
        // index adds 4 bytes per row; one exp per element
        const double n = double(a.rows) * double(a.cols);
        const double per = (MODE == kSoftmax || kLogSm) ? 8.0 : MODE == kCeIndex ? 4.0 : MODE == kCeOnehot ? 8.0
                         : (MODE == kCeBwdIndex || kBoth) ? 8.0 : 12.0;   // kCeBwdOnehot, kSoftmaxBwd: two inputs, one output
        const bool index = (MODE == kCeIndex || MODE == kCeBwdIndex || kBoth);
        account(per * n + (index ? 4.0 * double(a.rows) : 0.0), n);
    }
    ScratchUse use(stream, kLoss);
    if (kLoss) a.partials = reinterpret_cast<double*>(use.ptr());
    if (kLoss && !a.partials) return CTAMD_EINVAL;
    // rows are dealt to a chip-filling number of blocks (each walks several rows, prefetching the next)
    const size_t groups = (a.cols + 3) / 4;
    const int threads = groups <= 64 * 8 ? 64 : groups <= 256 * 8 ? 256 : 1024;
    size_t fill = size_t(compute_units() > 0 ? compute_units() : 256) * size_t(2048 / threads);
    if (fill > kMaxRowBlocks) fill = kMaxRowBlocks;
    if (kLoss && fill > 2048) fill = 2048;         // one partial per block: keep the fold of the partials short
    unsigned grid = a.rows < fill ? unsigned(a.rows) : unsigned(fill);
    bool vec = (a.cols % 4 == 0) && aligned16(a.x) &&
               (MODE == kSoftmax || kLogSm || MODE == kCeIndex || MODE == kCeBwdIndex || kBoth || aligned16(a.t)) &&
               (!kWrites || aligned16(a.out));
    if (MODE == kCeIndex && a.cols >= 2048) {
        size_t fill_online = size_t(compute_units() > 0 ? compute_units() : 256) * 8;
        grid = a.rows < fill_online ? unsigned(a.rows) : unsigned(fill_online);
        if (vec) hipLaunchKernelGGL((ce_index_online_kernel<true>), dim3(grid), dim3(256), 0, s, a);
        else hipLaunchKernelGGL((ce_index_online_kernel<false>), dim3(grid), dim3(256), 0, s, a);
        int rc0 = launched(name);
        if (rc0) return rc0;
        hipLaunchKernelGGL(loss_stage2, dim3(1), dim3(256), 0, s, a.partials, grid, loss_out, MODE == kCeIndex ? a.status : nullptr);
        return launched(name);
    }
    bool done = vec ? launch_resident<MODE_, 4>(a, grid, s) : launch_resident<MODE_, 1>(a, grid, s);
    if (!done) {
        if constexpr (kBoth)
            return fail(CTAMD_ERANGE, "%s: a row does not fit a block's registers (32768 columns, 8192 without 128-bit accesses): "
                        "use the separate forward and backward entry points", name);
        else if constexpr (MODE == kSoftmax || MODE == kSoftmaxBwd || MODE == kLogSoftmaxFast || MODE == kLogSoftmaxBwd) {
            if (vec && (a.cols >> 2) <= kKeepVectors) {
                // the kept operand takes 128 KiB of LDS: more than a kernel gets without asking, once per device
                constexpr size_t kKeepBytes = size_t(kKeepLds) * 1024 * sizeof(v4f);
                static bool raised[64] = {};
                int dev = 0;
                if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(CTAMD_EHIP, "%s: no current device", name);
                if (!raised[dev]) {
                    if (hipFuncSetAttribute(reinterpret_cast<const void*>(row_keep_kernel<MODE_>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            int(kKeepBytes)) != hipSuccess)
                        return fail(CTAMD_EHIP, "%s: the device does not give a block %zu bytes of LDS", name, kKeepBytes);
                    raised[dev] = true;
                }
                const unsigned cus = unsigned(compute_units() > 0 ? compute_units() : 256);
                hipLaunchKernelGGL((row_keep_kernel<MODE_>), dim3(grid < cus ? grid : cus), dim3(1024), kKeepBytes, s, a);
            } else if (vec) hipLaunchKernelGGL((row_stream_vec_kernel<MODE_>), dim3(grid), dim3(1024), 0, s, a);
            else hipLaunchKernelGGL((row_stream_kernel<MODE>), dim3(grid), dim3(1024), 0, s, a);
        } else
            hipLaunchKernelGGL((row_stream_kernel<MODE>), dim3(grid), dim3(1024), 0, s, a);
    }
    int rc = launched(name);
    if (rc) return rc;
    if (kLoss) {
        hipLaunchKernelGGL(loss_stage2, dim3(1), dim3(256), 0, s, a.partials, grid, loss_out, kIndexLoss ? a.status : nullptr);
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


// log_softmax along dim 0 and its gradient, one thread per column, rows in order (small matrices)
__global__ __launch_bounds__(256) void log_softmax_cols_kernel(const float* __restrict__ x, float* __restrict__ y,
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
    for (size_t i = 0; i < rows; ++i) s += cta_expf_tab(x[i * cols + j] - m, s_exp2);
    const float lg = cta_logf(s, cta_log_tab);
    for (size_t i = 0; i < rows; ++i) {
        const float d = x[i * cols + j] - m;
        y[i * cols + j] = d - lg;
    }
}
__global__ __launch_bounds__(256) void log_softmax_bwd_cols_kernel(const float* __restrict__ y, const float* __restrict__ g,
                                                                   float* __restrict__ dx, size_t rows, size_t cols) {
    __shared__ uint64_t s_exp2[32];
    stage_exp_table(s_exp2);
    size_t j = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (j >= cols) return;
    float d = 0.0f;
    for (size_t i = 0; i < rows; ++i) d += g[i * cols + j];
    for (size_t i = 0; i < rows; ++i) {
        const float t = cta_expf_tab(y[i * cols + j], s_exp2) * d;
        dx[i * cols + j] = g[i * cols + j] - t;
    }
}

// Tall matrices (128 rows or more): the column statistics as chunked reductions over rows, like the
// column sum - a block owns a strip of 256 * W columns and a chunk of rows and walks its rows in
// order, two rows in flight; per-chunk partials are folded by a second launch.  Forward: per chunk
// a running (max, sum of exp(x - max)) pair, rescaled when the maximum moves; the fold
// brings the chunks to the column maximum; then y = exp(x - max) / sum with the exact quotient (the
// exponential is recomputed rather than stored: 12 B/elem instead of 16).
// Backward: column dots of g and y, then dx = y * (g - dot).  The sums are chunked (fp32 inside a
// chunk, double across chunks) where the reference adds the rows one after the other: the same
// values to ~1e-7 relative, against 18 ms for a [16384 x 4096] matrix when one thread walks a
// whole column alone.
enum ColMode { kColOnline, kColSoftmaxOut, kColDot, kColBwdOut, kColSum, kColLogSoftmaxOut, kColLogBwdOut };

template <int MODE, int W, bool FAST>
__global__ __launch_bounds__(256) void col_walk_kernel(const float* __restrict__ x, const float* __restrict__ x2,
                                                       const float* __restrict__ p0, const float* __restrict__ p1,
                                                       float* __restrict__ out, size_t rows, size_t cols,
                                                       size_t rows_per_block) {
    __shared__ uint64_t s_exp2[32];
    if ((MODE == kColSoftmaxOut || MODE == kColLogBwdOut) && !FAST) stage_exp_table(s_exp2);
    const size_t col = (size_t(blockIdx.x) * 256 + threadIdx.x) * W;
    if (col >= cols) return;
    const size_t r0 = size_t(blockIdx.y) * rows_per_block;
    size_t r1 = r0 + rows_per_block;
    if (r1 > rows) r1 = rows;
    float a0[W], a1[W], q0[W];          // two accumulators (even / odd rows of the chunk); per-column parameter
    float m0[W], m1[W];                 // kColOnline: the running maxima that a0 / a1 are relative to
    double rcp[W];
#pragma unroll
    for (int e = 0; e < W; ++e) {
        a0[e] = a1[e] = 0.0f;
        m0[e] = m1[e] = kNegInf;
        q0[e] = (MODE == kColSoftmaxOut || MODE == kColBwdOut || MODE == kColLogSoftmaxOut || MODE == kColLogBwdOut) ? p0[col + e] : 0.0f;
        rcp[e] = (MODE == kColSoftmaxOut) ? 1.0 / double(p1[col + e]) : 0.0;
    }
    float rcp_f[W];                     // FAST: e * (1 / sum)
#pragma unroll
    for (int e = 0; e < W; ++e) rcp_f[e] = (MODE == kColSoftmaxOut && FAST) ? 1.0f / p1[col + e] : 0.0f;
    float lg[W];                        // kColLogSoftmaxOut: log of the column's sum
#pragma unroll
    for (int e = 0; e < W; ++e) lg[e] = (MODE == kColLogSoftmaxOut) ? cta_logf(p1[col + e], cta_log_tab) : 0.0f;
    auto load = [&](const float* __restrict__ base, size_t r, float (&v)[W]) {
        if (W == 4) {
            // the writing passes read their operands for the last time: streaming hint (on the reading
            // passes it costs the second pass its cache hits: 152 -> 162 us at [16384 x 4096])
            constexpr bool kLast = (MODE == kColSoftmaxOut || MODE == kColBwdOut || MODE == kColLogSoftmaxOut || MODE == kColLogBwdOut);
            v4f t = kLast ? __builtin_nontemporal_load(reinterpret_cast<const v4f*>(base + r * cols + col))
                          : *reinterpret_cast<const v4f*>(base + r * cols + col);
#pragma unroll
            for (int e = 0; e < W; ++e) v[e] = t[e];
        } else {
            v[0] = base[r * cols + col];
        }
    };
    auto store = [&](size_t r, const float (&v)[W]) {
        if (W == 4) {
            v4f t;
#pragma unroll
            for (int e = 0; e < W; ++e) t[e] = v[e];
            // always with the streaming hint: the pass that writes re-reads x, and what the memory-side cache
            // still holds of x from the pass before must not be pushed out by the result (139 against 161 us)
            __builtin_nontemporal_store(t, reinterpret_cast<v4f*>(out + r * cols + col));
        } else {
            out[r * cols + col] = v[0];
        }
    };
    auto one_row = [&](size_t r, float (&acc)[W], float (&mx)[W], const float (&v)[W], const float (&w)[W]) {
        float o[W];
#pragma unroll
        for (int e = 0; e < W; ++e) {
            if (MODE == kColOnline) {
                // one exponential per element either way, without a branch: of the old maximum's
                // distance when the maximum moves (the sum is rescaled; exp(-inf) = 0 at the first
                // row), of the element's distance otherwise (an element of -inf adds nothing)
                // (the hardware exponential: only the column sum is formed from it, ~1e-7 relative)
                const bool up = v[e] > mx[e];
                float ex = __builtin_amdgcn_exp2f((up ? mx[e] - v[e] : v[e] - mx[e]) * kLog2e);
                ex = v[e] == kNegInf ? 0.0f : ex;
                acc[e] = up ? __fmaf_rn(acc[e], ex, 1.0f) : acc[e] + ex;
                mx[e] = up ? v[e] : mx[e];
            } else if (MODE == kColSoftmaxOut) {
                o[e] = FAST ? cta_exp_hw_nonpos(v[e] - q0[e]) * rcp_f[e] : cta_div_rcp(cta_expf_nonpos(v[e] - q0[e], s_exp2), rcp[e]);
            }
            else if (MODE == kColDot) acc[e] = __fmaf_rn(w[e], v[e], acc[e]);
            else if (MODE == kColSum) acc[e] += v[e];
            else if (MODE == kColLogSoftmaxOut) {
                const float d = v[e] - q0[e];
                o[e] = d - lg[e];
            } else if (MODE == kColLogBwdOut) {                  // v = y, w = g, q0 = column sum of g
                const float t = (FAST ? cta_exp_hw(v[e]) : cta_expf_tab(v[e], s_exp2)) * q0[e];
                o[e] = w[e] - t;
            } else o[e] = v[e] * (w[e] - q0[e]);
        }
        if (MODE == kColSoftmaxOut || MODE == kColBwdOut || MODE == kColLogSoftmaxOut || MODE == kColLogBwdOut) store(r, o);
    };
    constexpr bool kTwo = (MODE == kColDot || MODE == kColBwdOut || MODE == kColLogBwdOut);     // x = y, x2 = g
    size_t r = r0;
    constexpr int kRows = 4;                // rows whose loads are in flight before the first is used (8: no gain)
    for (; r + kRows <= r1; r += kRows) {
        float v[kRows][W], w[kRows][W] = {};
#pragma unroll
        for (int i = 0; i < kRows; ++i) load(x, r + i, v[i]);
        if (kTwo) {
#pragma unroll
            for (int i = 0; i < kRows; ++i) load(x2, r + i, w[i]);
        }
#pragma unroll
        for (int i = 0; i < kRows; i += 2) {
            one_row(r + i, a0, m0, v[i], w[i]);
            one_row(r + i + 1, a1, m1, v[i + 1], w[i + 1]);
        }
    }
    for (; r < r1; ++r) {
        float v0[W], w0[W] = {};
        load(x, r, v0);
        if (kTwo) load(x2, r, w0);
        if ((r - r0) & 1) one_row(r, a1, m1, v0, w0);
        else one_row(r, a0, m0, v0, w0);
    }
    if (MODE == kColDot || MODE == kColSum) {
#pragma unroll
        for (int e = 0; e < W; ++e) out[size_t(blockIdx.y) * cols + col + e] = a0[e] + a1[e];
    }
    if (MODE == kColOnline) {
        // the chunk's pair: both halves brought to the larger maximum; maxima in the first
        // gridDim.y partial rows, sums in the next gridDim.y
#pragma unroll
        for (int e = 0; e < W; ++e) {
            const float m = m1[e] > m0[e] ? m1[e] : m0[e];
            float sum = 0.0f;
            if (m0[e] != kNegInf) sum += a0[e] * __builtin_amdgcn_exp2f((m0[e] - m) * kLog2e);
            if (m1[e] != kNegInf) sum += a1[e] * __builtin_amdgcn_exp2f((m1[e] - m) * kLog2e);
            out[size_t(blockIdx.y) * cols + col + e] = m;
            out[(size_t(gridDim.y) + blockIdx.y) * cols + col + e] = sum;
        }
    }
}

// The `chunks` partial rows of a column folded in double.  A block folds 32 columns; its 8 groups
// of 32 lanes take every 8th chunk and are added in group order.
constexpr int kFoldCols = 32, kFoldGroups = 8;
__global__ __launch_bounds__(256) void col_fold_kernel(const float* __restrict__ partials, float* __restrict__ out, size_t cols,
                                                       unsigned chunks) {
    __shared__ double s_t[kFoldGroups][kFoldCols];
    const unsigned lane = threadIdx.x % kFoldCols, group = threadIdx.x / kFoldCols;
    const size_t c = size_t(blockIdx.x) * kFoldCols + lane;
    const bool live = c < cols;
    double t = 0.0;
    if (live) {
#pragma unroll 4
        for (unsigned k = group; k < chunks; k += kFoldGroups) t += double(partials[size_t(k) * cols + c]);
    }
    s_t[group][lane] = t;
    __syncthreads();
    if (group == 0 && live) {
        double sum = 0.0;
#pragma unroll
        for (int g = 0; g < kFoldGroups; ++g) sum += s_t[g][lane];
        out[c] = float(sum);
    }
}

// The (max, sum) pairs of the online column pass (maxima in the first `chunks` rows of partials,
// sums in the next) brought to the column maximum, out_max[c], and added in double, out[c].  A CU
// draws only some tens of GB/s by itself, so the fold is spread over as many blocks as the columns
// allow: a block folds 16 columns, its 64 groups of 16 lanes take every 64th chunk (four loads in
// flight each), and the groups' maxima and sums are combined through LDS in group order.  (32
// columns x 8 groups on 128 blocks, or 64 columns x 16 groups on 64 blocks, took 18.5 us for the
// 8 MiB of partials of a [16384 x 4096] matrix, an eighth of the whole softmax.)
constexpr int kPairCols = 16, kPairGroups = 64, kPairAhead = 4;
__global__ __launch_bounds__(kPairCols * kPairGroups) void col_fold_pairs_kernel(const float* __restrict__ partials,
                                                                                 float* __restrict__ out_max, float* __restrict__ out,
                                                                                 size_t cols, unsigned chunks) {
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_m[kPairGroups][kPairCols];
    __shared__ double s_t[kPairGroups][kPairCols];
    stage_exp_table(s_exp2);
    const unsigned lane = threadIdx.x % kPairCols, group = threadIdx.x / kPairCols;
    const size_t c = size_t(blockIdx.x) * kPairCols + lane;
    const bool live = c < cols;
    float m = kNegInf;
    for (unsigned k0 = group; k0 < chunks; k0 += kPairGroups * kPairAhead) {
        float mk[kPairAhead];
#pragma unroll
        for (int i = 0; i < kPairAhead; ++i) {
            const unsigned k = k0 + unsigned(i) * kPairGroups;
            mk[i] = (live && k < chunks) ? partials[size_t(k) * cols + c] : kNegInf;
        }
#pragma unroll
        for (int i = 0; i < kPairAhead; ++i) m = mk[i] > m ? mk[i] : m;
    }
    s_m[group][lane] = m;
    __syncthreads();
#pragma unroll
    for (int g = 0; g < kPairGroups; ++g) m = s_m[g][lane] > m ? s_m[g][lane] : m;
    double t = 0.0;
    for (unsigned k0 = group; k0 < chunks; k0 += kPairGroups * kPairAhead) {
        float mk[kPairAhead], sk[kPairAhead];
#pragma unroll
        for (int i = 0; i < kPairAhead; ++i) {
            const unsigned k = k0 + unsigned(i) * kPairGroups;
            const bool in = live && k < chunks;
            mk[i] = in ? partials[size_t(k) * cols + c] : kNegInf;
            sk[i] = in ? partials[(size_t(chunks) + k) * cols + c] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < kPairAhead; ++i)
            if (mk[i] != kNegInf) t += double(sk[i]) * double(cta_expf_nonpos(mk[i] - m, s_exp2));
    }
    s_t[group][lane] = t;
    __syncthreads();
    if (group == 0 && live) {
        double sum = 0.0;
#pragma unroll
        for (int g = 0; g < kPairGroups; ++g) sum += s_t[g][lane];
        out_max[c] = m;
        out[c] = float(sum);
    }
}

struct ColPlan {
    size_t rows_per_block, chunks;
    dim3 grid;
    float* partials;
    float* v0;      // [cols]
    float* v1;      // [cols]
    bool vec;
};
// false: the matrix is small (the sequential kernels serve it) or does not fit the scratch layout
bool plan_cols(size_t rows, size_t cols, bool aligned, ColPlan& p, void* stream) {
    if (rows < 128) return false;
    float* sc = scratch();                 // claimed for `stream` by the caller (a ScratchUse in its scope)
    if (!sc) return false;
    size_t chunks = (rows + 31) / 32;
    if (chunks > 256) chunks = 256;
    if ((2 * chunks + 2) * cols > kScratchFloats) {             // two partial rows per chunk (forward), two vectors
        if (4 * cols > kScratchFloats) return false;
        chunks = (kScratchFloats / cols - 2) / 2;
    }
    p.rows_per_block = (rows + chunks - 1) / chunks;
    p.chunks = (rows + p.rows_per_block - 1) / p.rows_per_block;
    p.vec = aligned && cols % 4 == 0;
    const size_t per_block = size_t(256) * (p.vec ? 4 : 1);
    const size_t strips = (cols + per_block - 1) / per_block;
    if (strips > 0x7fffffffu || p.chunks > 65535) return false;
    p.grid = dim3(unsigned(strips), unsigned(p.chunks));
    p.partials = sc;
    p.v0 = sc + 2 * p.chunks * cols;
    p.v1 = p.v0 + cols;
    return true;
}

template <int MODE, bool FAST = false>
void launch_col_walk(const ColPlan& p, const float* x, const float* x2, const float* p0, const float* p1, float* out, size_t rows,
                     size_t cols, hipStream_t s) {
    if (p.vec) hipLaunchKernelGGL((col_walk_kernel<MODE, 4, FAST>), p.grid, dim3(256), 0, s, x, x2, p0, p1, out, rows, cols, p.rows_per_block);
    else hipLaunchKernelGGL((col_walk_kernel<MODE, 1, FAST>), p.grid, dim3(256), 0, s, x, x2, p0, p1, out, rows, cols, p.rows_per_block);
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols, void* stream) {
    Args a{x, nullptr, nullptr, y, nullptr, nullptr, nullptr, rows, cols, nullptr, nullptr};
    if (fast_math()) return run_rows<kSoftmaxFast>(__func__, a, nullptr, stream);
    return run_rows<kSoftmax>(__func__, a, nullptr, stream);
}
int ctamd_cross_entropy_onehot_f32(const float* x, const float* t, float* out, size_t rows, size_t cols, void* stream) {
    Args a{x, t, nullptr, nullptr, nullptr, nullptr, nullptr, rows, cols, nullptr, nullptr};
    return run_rows<kCeOnehot>(__func__, a, out, stream);
}
int ctamd_cross_entropy_index_f32(const float* x, const float* idx, float* out, int32_t* status, size_t rows,
                                  size_t cols, void* stream) {
    return ctamd_cross_entropy_index_stats_f32(x, idx, out, status, nullptr, rows, cols, stream);
}
int ctamd_cross_entropy_backward_index_stats_f32(const float* x, const float* idx, const float* stats, const float* g1,
                                                 float* dx, size_t rows, size_t cols, void* stream) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!x || !idx || !stats || !g1 || !dx) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    if (rows > (size_t(1) << 62) / cols) return fail(CTAMD_ERANGE, "%s: rows*cols overflows", __func__);
    if (cols > size_t(0x7fffffff)) return fail(CTAMD_ERANGE, "%s: more than 2^31-1 columns", __func__);
    Args a{x, idx, g1, dx, nullptr, nullptr, const_cast<float*>(stats), rows, cols, nullptr, nullptr};
    const size_t fill = size_t(compute_units() > 0 ? compute_units() : 256) * 8;
    const unsigned grid = rows < fill ? unsigned(rows) : unsigned(fill);
    const bool vec = (cols % 4 == 0) && aligned16(x) && aligned16(dx);
    if (vec && (cols >= 2048 || fast_math())) hipLaunchKernelGGL((ce_bwd_stats_kernel<true, true>), dim3(grid), dim3(256), 0, as_stream(stream), a);
    else if (vec) hipLaunchKernelGGL((ce_bwd_stats_kernel<true, false>), dim3(grid), dim3(256), 0, as_stream(stream), a);
    else hipLaunchKernelGGL((ce_bwd_stats_kernel<false, false>), dim3(grid), dim3(256), 0, as_stream(stream), a);
    account(8.0 * double(rows) * double(cols) + 12.0 * double(rows), double(rows) * double(cols));
    return launched(__func__);
}
int ctamd_cross_entropy_index_stats_f32(const float* x, const float* idx, float* out, int32_t* status, float* stats,
                                        size_t rows, size_t cols, void* stream) {
    Args a{x, idx, nullptr, nullptr, nullptr, status, stats, rows, cols, nullptr, nullptr};
    return run_rows<kCeIndex>(__func__, a, out, stream);
}
int ctamd_cross_entropy_index_fused_f32(const float* x, const float* idx, float* out, int32_t* status, float* dx, size_t rows,
                                        size_t cols, void* stream) {
    Args a{x, idx, nullptr, dx, nullptr, status, nullptr, rows, cols, nullptr, nullptr};
    // long rows use the hardware exponential throughout, as the forward / backward-from-statistics
    // pair does (<= 2e-7 from the exact form)
    if (cols >= 2048 || fast_math()) return run_rows<kCeIndexBothFast>(__func__, a, out, stream);
    return run_rows<kCeIndexBoth>(__func__, a, out, stream);
}
int ctamd_cross_entropy_backward_onehot_f32(const float* x, const float* t, const float* g1, float* dx, size_t rows,
                                            size_t cols, void* stream) {
    Args a{x, t, g1, dx, nullptr, nullptr, nullptr, rows, cols, nullptr, nullptr};
    if (fast_math()) return run_rows<kCeBwdOnehotFast>(__func__, a, nullptr, stream);
    return run_rows<kCeBwdOnehot>(__func__, a, nullptr, stream);
}
int ctamd_cross_entropy_backward_index_f32(const float* x, const float* idx, const float* g1, float* dx, size_t rows,
                                           size_t cols, void* stream) {
    Args a{x, idx, g1, dx, nullptr, nullptr, nullptr, rows, cols, nullptr, nullptr};
    if (fast_math()) return run_rows<kCeBwdIndexFast>(__func__, a, nullptr, stream);
    return run_rows<kCeBwdIndex>(__func__, a, nullptr, stream);
}
int ctamd_softmax_backward_rows_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream) {
    Args a{y, g, nullptr, dx, nullptr, nullptr, nullptr, rows, cols, nullptr, nullptr};
    return run_rows<kSoftmaxBwd>(__func__, a, nullptr, stream);
}

int ctamd_log_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols, void* stream) {
    Args a{x, nullptr, nullptr, y, nullptr, nullptr, nullptr, rows, cols, nullptr, nullptr};
    if (cols >= 2048) return run_rows<kLogSoftmaxFast>(__func__, a, nullptr, stream);
    return run_rows<kLogSoftmax>(__func__, a, nullptr, stream);
}
int ctamd_log_softmax_backward_rows_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream) {
    Args a{y, g, nullptr, dx, nullptr, nullptr, nullptr, rows, cols, nullptr, nullptr};
    if (fast_math()) return run_rows<kLogSoftmaxBwdFast>(__func__, a, nullptr, stream);
    return run_rows<kLogSoftmaxBwd>(__func__, a, nullptr, stream);
}
int ctamd_log_softmax_cols_f32(const float* x, float* y, size_t rows, size_t cols, void* stream) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!x || !y) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    ScratchUse use(stream, rows >= 128);
    if (rows >= 128 && !use.ptr()) return CTAMD_EINVAL;
    ColPlan p;
    account(8.0 * double(rows) * double(cols), double(rows) * double(cols));
    if (plan_cols(rows, cols, aligned16(x) && aligned16(y), p, stream)) {
        hipStream_t s = as_stream(stream);
        launch_col_walk<kColOnline>(p, x, nullptr, nullptr, nullptr, p.partials, rows, cols, s);
        hipLaunchKernelGGL(col_fold_pairs_kernel, dim3(unsigned((cols + kPairCols - 1) / kPairCols)), dim3(kPairCols * kPairGroups), 0, s, p.partials, p.v0, p.v1, cols, unsigned(p.chunks));
        launch_col_walk<kColLogSoftmaxOut>(p, x, nullptr, p.v0, p.v1, y, rows, cols, s);
        return launched(__func__);
    }
    hipLaunchKernelGGL(log_softmax_cols_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, as_stream(stream), x, y, rows, cols);
    return launched(__func__);
}
int ctamd_log_softmax_backward_cols_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!y || !g || !dx) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    ScratchUse use(stream, rows >= 128);
    if (rows >= 128 && !use.ptr()) return CTAMD_EINVAL;
    ColPlan p;
    account(12.0 * double(rows) * double(cols), 2.0 * double(rows) * double(cols));
    if (plan_cols(rows, cols, aligned16(y) && aligned16(g) && aligned16(dx), p, stream)) {
        hipStream_t s = as_stream(stream);
        launch_col_walk<kColSum>(p, g, nullptr, nullptr, nullptr, p.partials, rows, cols, s);
        hipLaunchKernelGGL(col_fold_kernel, dim3(unsigned((cols + kFoldCols - 1) / kFoldCols)), dim3(256), 0, s, p.partials, p.v0,
                           cols, unsigned(p.chunks));
        if (fast_math()) launch_col_walk<kColLogBwdOut, true>(p, y, g, p.v0, nullptr, dx, rows, cols, s);
        else launch_col_walk<kColLogBwdOut>(p, y, g, p.v0, nullptr, dx, rows, cols, s);
        return launched(__func__);
    }
    hipLaunchKernelGGL(log_softmax_bwd_cols_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, as_stream(stream), y, g, dx, rows, cols);
    return launched(__func__);
}

int ctamd_softmax_cols_f32(const float* x, float* y, size_t rows, size_t cols, void* stream) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!x || !y) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    ScratchUse use(stream, rows >= 128);
    if (rows >= 128 && !use.ptr()) return CTAMD_EINVAL;
    ColPlan p;
    if (plan_cols(rows, cols, aligned16(x) && aligned16(y), p, stream)) {
        hipStream_t s = as_stream(stream);
        launch_col_walk<kColOnline>(p, x, nullptr, nullptr, nullptr, p.partials, rows, cols, s);
        hipLaunchKernelGGL(col_fold_pairs_kernel, dim3(unsigned((cols + kPairCols - 1) / kPairCols)), dim3(kPairCols * kPairGroups), 0, s, p.partials, p.v0, p.v1, cols, unsigned(p.chunks));
        if (fast_math()) launch_col_walk<kColSoftmaxOut, true>(p, x, nullptr, p.v0, p.v1, y, rows, cols, s);
        else launch_col_walk<kColSoftmaxOut>(p, x, nullptr, p.v0, p.v1, y, rows, cols, s);
        account(8.0 * double(rows) * double(cols), double(rows) * double(cols));
        return launched(__func__);
    }
    hipLaunchKernelGGL(softmax_cols_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, as_stream(stream), x, y,
                       rows, cols);
    account(8.0 * double(rows) * double(cols), double(rows) * double(cols));
    return launched(__func__);
}
int ctamd_softmax_backward_cols_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream) {
    if (rows == 0 || cols == 0) return CTAMD_OK;
    if (!y || !g || !dx) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    ScratchUse use(stream, rows >= 128);
    if (rows >= 128 && !use.ptr()) return CTAMD_EINVAL;
    ColPlan p;
    if (plan_cols(rows, cols, aligned16(y) && aligned16(g) && aligned16(dx), p, stream)) {
        hipStream_t s = as_stream(stream);
        launch_col_walk<kColDot>(p, y, g, nullptr, nullptr, p.partials, rows, cols, s);
        hipLaunchKernelGGL(col_fold_kernel, dim3(unsigned((cols + kFoldCols - 1) / kFoldCols)), dim3(256), 0, s, p.partials, p.v0,
                           cols, unsigned(p.chunks));
        launch_col_walk<kColBwdOut>(p, y, g, p.v0, nullptr, dx, rows, cols, s);
        account(12.0 * double(rows) * double(cols), 2.0 * double(rows) * double(cols));
        return launched(__func__);
    }
    hipLaunchKernelGGL(softmax_bwd_cols_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, as_stream(stream), y,
                       g, dx, rows, cols);
    account(12.0 * double(rows) * double(cols), 2.0 * double(rows) * double(cols));
    return launched(__func__);
}

}  // extern "C"
