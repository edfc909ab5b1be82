// The data side of the reference's MNIST demo on the device: IDX pixel bytes -> fp32 in [0, 1],
// class labels -> one-hot rows, and the accuracy count.  Byte- and index-shaped work bound by HBM.
#include "common.h"
#include "devmath.h"

namespace ctamd {
namespace {

constexpr int kThreads = 256;
typedef float v4f __attribute__((ext_vector_type(4)));

// dst[i] = src[i] / 255.0f.  A thread converts four groups of 4 pixels, 256 groups apart: each 32-bit
// load and each 128-bit store of a wave covers one contiguous run (one thread converting 16
// neighbouring pixels scatters its four stores over four cache lines: 1.7 TB/s against 5 here).
// The division goes through the exact double reciprocal (cta_div_rcp): same bits as the IEEE
// quotient, without the division sequence.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void u8_to_unit_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst,
                                                              size_t n) {
    const double rcp = 1.0 / 255.0;
    if (VEC) {
        constexpr int U = 4;
        const size_t n4 = n / 4;
        const size_t base = size_t(blockIdx.x) * (kThreads * U) + threadIdx.x;
        uint32_t w[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t i = base + size_t(u) * kThreads;
            if (i < n4) w[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(src) + i);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t i = base + size_t(u) * kThreads;
            if (i < n4) {
                v4f o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = cta_div_rcp(float((w[u] >> (8 * e)) & 0xffu), rcp);
                __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(dst) + i);
            }
        }
    } else {
        const size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x;
        if (i < n) dst[i] = cta_div_rcp(float(src[i]), rcp);
    }
}

// out[i, j] = (j == int(labels[i])) ? 1 : 0; one thread per element, rows * classes < 2^63.
__global__ __launch_bounds__(kThreads) void onehot_kernel(const float* __restrict__ labels, float* __restrict__ out,
                                                          size_t rows, size_t classes) {
    const size_t stride = size_t(gridDim.x) * kThreads;
    for (size_t idx = size_t(blockIdx.x) * kThreads + threadIdx.x; idx < rows * classes; idx += stride) {
        const size_t i = idx / classes, j = idx - i * classes;
        out[idx] = (int64_t(j) == int64_t(class_index(labels[i]))) ? 1.0f : 0.0f;
    }
}

__global__ void clear_count(int32_t* p) { p[0] = 0; }

// One thread per row: the first index whose value exceeds all earlier ones, starting from -1.0f at
// index 0, compared with int(label); per-block popcount, one integer atomic per block.
__global__ __launch_bounds__(kThreads) void count_correct_kernel(const float* __restrict__ pred,
                                                                 const float* __restrict__ labels,
                                                                 int32_t* __restrict__ count, size_t rows,
                                                                 size_t classes) {
    __shared__ int s_hits;
    if (threadIdx.x == 0) s_hits = 0;
    __syncthreads();
    const size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x;
    int hit = 0;
    if (i < rows) {
        const float* __restrict__ p = pred + i * classes;
        int best = 0;
        float mx = -1.0f;
        for (size_t j = 0; j < classes; ++j) {
            float v = p[j];
            if (v > mx) {
                mx = v;
                best = int(j);
            }
        }
        hit = (best == class_index(labels[i])) ? 1 : 0;
    }
    const int wave_hits = __popcll(__ballot(hit));
    if ((threadIdx.x & 63) == 0 && wave_hits) atomicAdd(&s_hits, wave_hits);
    __syncthreads();
    if (threadIdx.x == 0 && s_hits) atomicAdd(count, s_hits);
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" {

int ctamd_u8_to_unit_f32(const uint8_t* src, float* dst, size_t n, void* stream) {
    if (n == 0) return CTAMD_OK;
    if (!src || !dst) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    hipStream_t s = as_stream(stream);
    const bool vec = (n % 4 == 0) && (reinterpret_cast<uintptr_t>(src) & 3u) == 0 && aligned16(dst);
    const size_t per_block = vec ? size_t(kThreads) * 16 : size_t(kThreads);
    const size_t blocks = (n + per_block - 1) / per_block;
    if (blocks > 0x7fffffffu) return fail(CTAMD_ERANGE, "%s: too many elements", __func__);
    if (vec) hipLaunchKernelGGL(u8_to_unit_kernel<true>, dim3(unsigned(blocks)), dim3(kThreads), 0, s, src, dst, n);
    else hipLaunchKernelGGL(u8_to_unit_kernel<false>, dim3(unsigned(blocks)), dim3(kThreads), 0, s, src, dst, n);
    account(5.0 * double(n), double(n));
    return launched(__func__);
}

int ctamd_onehot_f32(const float* labels, float* out, size_t rows, size_t classes, void* stream) {
    if (rows == 0 || classes == 0) return CTAMD_OK;
    if (!labels || !out) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    if (rows > (size_t(1) << 62) / classes) return fail(CTAMD_ERANGE, "%s: rows*classes overflows", __func__);
    hipLaunchKernelGGL(onehot_kernel, dim3(stream_grid(rows * classes, kThreads)), dim3(kThreads), 0, as_stream(stream),
                       labels, out, rows, classes);
    account(4.0 * double(rows) * double(classes) + 4.0 * double(rows), 0.0);
    return launched(__func__);
}

int ctamd_count_correct_f32(const float* pred, const float* labels, int32_t* count, size_t rows, size_t classes,
                            void* stream) {
    if (!count) return fail(CTAMD_EINVAL, "%s: null output", __func__);
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(clear_count, dim3(1), dim3(1), 0, s, count);
    int rc = launched(__func__);
    if (rc || rows == 0) return rc;
    if (!pred || !labels) return fail(CTAMD_EINVAL, "%s: null input", __func__);
    if (classes == 0) return fail(CTAMD_EINVAL, "%s: zero classes", __func__);
    const size_t blocks = (rows + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffu || rows > size_t(0x7fffffff)) return fail(CTAMD_ERANGE, "%s: too many rows", __func__);
    hipLaunchKernelGGL(count_correct_kernel, dim3(unsigned(blocks)), dim3(kThreads), 0, s, pred, labels, count, rows,
                       classes);
    account(4.0 * double(rows) * double(classes) + 4.0 * double(rows), 0.0);
    return launched(__func__);
}

}  // extern "C"
