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

// ---- Stage 1 of the two-stage column sum of a narrow matrix (a row is at most 128 vectors), shared
// by the column-sum entry point and by the tiled product, which can carry the sums of its second
// operand along as extra blocks of its launches: the same code on the same partition, hence the same bits.
constexpr int kFoldLanes = 4;        // lanes per column in stage 2

struct ColsumNarrowPlan {
    unsigned lanes;                  // vectors per row
    unsigned groups;                 // row groups of a block
    size_t rows_per_block;
    unsigned chunks;                 // blocks of stage 1 = partial rows
};
// false: the matrix is not narrow (the strip kernels sum it)
inline bool colsum_narrow_plan(size_t rows, size_t cols, bool vec, ColsumNarrowPlan* plan) {
    const size_t lanes = cols / (vec ? 4 : 1);
    if (lanes > 128 || lanes == 0) return false;
    const size_t groups = kColsumThreads / lanes;
    size_t rows_per_block = groups * 8;                         // eight rows per thread, four in flight
    size_t chunks = (rows + rows_per_block - 1) / rows_per_block;
    if (chunks > 256) {
        rows_per_block = (rows + 255) / 256;
        chunks = (rows + rows_per_block - 1) / rows_per_block;
    }
    plan->lanes = unsigned(lanes); plan->groups = unsigned(groups); plan->rows_per_block = rows_per_block; plan->chunks = unsigned(chunks);
    return true;
}

// A block's threads form `groups` row groups; group k walks rows k, k + groups, ... of the block's
// chunk with four rows in flight, so the block reads its chunk as one contiguous run; the groups are
// added through LDS in group order and the block writes one partial row.  Every thread of the calling
// block must call (one barrier inside); the first kColsumThreads take part.  s_part: kColsumThreads * W floats.
template <bool VEC>
__device__ __forceinline__ void colsum_narrow_body(const float* __restrict__ g, float* __restrict__ partials, size_t rows, size_t cols,
                                                   unsigned lanes, unsigned groups, size_t rows_per_block, unsigned block,
                                                   unsigned thread, float* __restrict__ s_part) {
    typedef float vec4 __attribute__((ext_vector_type(4)));
    constexpr int W = VEC ? 4 : 1;
    const bool active = thread < unsigned(kColsumThreads);
    const unsigned lane = thread % lanes, group = thread / lanes;
    const size_t r0 = size_t(block) * rows_per_block;
    size_t r1 = r0 + rows_per_block;
    if (r1 > rows) r1 = rows;
    float acc[4][W];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int e = 0; e < W; ++e) acc[p][e] = 0.0f;
    if (active && group < groups) {
        const float* col = g + size_t(lane) * W;
        size_t r = r0 + group;
        for (; r + 3 * size_t(groups) < r1; r += 4 * size_t(groups)) {
            float x[4][W];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float* src = col + (r + size_t(p) * groups) * cols;
                if (VEC) {
                    vec4 t = *reinterpret_cast<const vec4*>(src);
#pragma unroll
                    for (int e = 0; e < W; ++e) x[p][e] = t[e];
                } else {
                    x[p][0] = *src;
                }
            }
#pragma unroll
            for (int p = 0; p < 4; ++p)
#pragma unroll
                for (int e = 0; e < W; ++e) acc[p][e] += x[p][e];
        }
        for (; r < r1; r += groups) {
            const float* src = col + r * cols;
#pragma unroll
            for (int e = 0; e < W; ++e) acc[0][e] += src[e];
        }
    }
    if (active) {
#pragma unroll
        for (int e = 0; e < W; ++e) s_part[thread * W + e] = (acc[0][e] + acc[1][e]) + (acc[2][e] + acc[3][e]);
    }
    __syncthreads();
    if (active && group == 0) {
        float t[W];
#pragma unroll
        for (int e = 0; e < W; ++e) t[e] = s_part[lane * W + e];
        for (unsigned k = 1; k < groups; ++k)
#pragma unroll
            for (int e = 0; e < W; ++e) t[e] += s_part[(k * lanes + lane) * W + e];
#pragma unroll
        for (int e = 0; e < W; ++e) partials[size_t(block) * cols + size_t(lane) * W + e] = t[e];
    }
}

}  // namespace ctamd

#endif
