// The column sum of a small matrix (a bias gradient of a few hundred rows) in one launch: rows
// added in double, kSmallLanes lanes per column, every lane its rows in order with eight loads in
// flight, the lanes of a column folded in lane order.  The body is shared by the column-sum entry
// point and by the small-product kernel, which can carry the sums of its second operand along as
// extra blocks of its own launch: the same code on the same partition, hence the same bits.
#ifndef CTAMD_COLSUM_SMALL_H
#define CTAMD_COLSUM_SMALL_H

#include <cstddef>
#include <hip/hip_runtime.h>

namespace ctamd {

constexpr int kColsumThreads = 256;
constexpr int kSmallLanes = 16;      // lanes per column when a small matrix is summed in one launch

// shapes the one-launch form takes
inline bool colsum_is_small(size_t rows, size_t cols) { return rows <= 1024 && rows * cols <= (size_t(1) << 19); }
inline unsigned colsum_small_blocks(size_t cols) {
    constexpr size_t kCols = kColsumThreads / kSmallLanes;
    return unsigned((cols + kCols - 1) / kCols);
}

// out[c] = sum over the `chunks` rows of partials[., c] for the columns of block `block`, LANES lanes
// per column.  Every thread of the calling block must call (one barrier inside); only the first
// kColsumThreads, `thread` < kColsumThreads, take part.  s_acc: kColsumThreads doubles of LDS.
template <int LANES>
__device__ __forceinline__ void colsum_fold_body(const float* __restrict__ partials, float* __restrict__ out, size_t cols,
                                                 unsigned chunks, unsigned block, unsigned thread, double* s_acc) {
    constexpr int TX = kColsumThreads / LANES;
    const bool active = thread < unsigned(kColsumThreads);
    const int tx = int(thread % TX), ty = int(thread / TX);
    const size_t c = size_t(block) * TX + tx;
    double acc = 0.0;
    if (active && c < cols) {
        unsigned k = unsigned(ty);
        for (; k + 7 * LANES < chunks; k += 8 * LANES) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partials[size_t(k + u * LANES) * cols + c];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += double(v[u]);
        }
        for (; k < chunks; k += LANES) acc += double(partials[size_t(k) * cols + c]);
    }
    if (active) s_acc[ty * TX + tx] = acc;
    __syncthreads();
    if (active && ty == 0 && c < cols) {
        double t = 0.0;
#pragma unroll
        for (int y = 0; y < LANES; ++y) t += s_acc[y * TX + tx];
        out[c] = float(t);
    }
}

}  // namespace ctamd

#endif
