// fp32 MatMul on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), fp32 accumulation.
//
// C[m,n] = sum_k A[m,k] * B[k,n] for operands given by element strides.  Every operand with a
// unit stride in one dimension is one of two tile kinds:
//   K-contiguous  (A row-major, or B given as a transposed view): tile kept in LDS as [rows][BK],
//                 fragments read with one 128-bit LDS load per 32x32 MFMA tile and 8-wide k chunk;
//   X-contiguous  (A given as a transposed view, or B row-major): tile kept as [BK][cols],
//                 fragments read with four 32-bit LDS loads.
// Within an 8-wide k chunk, lane half h (lane / 32) owns k = 4h .. 4h+3 for both operands - the
// sum over k is order-free, so the MFMA's (lane / 32) k index is simply re-labelled; that lets
// the K-contiguous kind fetch four consecutive k with a single load.
// One block (8 waves for the 256 x 256 tile, 4 for the 128 x 128 one) computes a BM x BN tile of C;
// global -> register -> LDS staging is double buffered so the loads of tile t+1 are in flight while
// tile t is multiplied, with one barrier per k tile.  Blocks are renumbered so that each XCD (blocks are
// dealt round-robin to the 8 XCDs) works on a compact band of C and re-uses its operand tiles
// from its own L2.  The tiles of the last, partly filled round of blocks - all tiles of a skinny
// output with a long K (the weight gradients of a small layer) - are cut along K into parts, one
// block each, so that they fill the chip; the parts go to the device scratch and a second launch
// adds them in a fixed order, so results stay deterministic.
//
// Two families of products do not go through those tiles (matmul_impl picks): a product of at most
// one 32 x 32 tile per CU with a short K (gemm_micro: the waves of a block share out K and feed the
// MFMAs from global memory directly), and a product with at most 16 output columns
// (gemm_narrow_rows / gemm_narrow_cols: fp32 FMAs on the vector units, A streamed once).
#include "colsum_small.h"
#include "common.h"


namespace ctamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kXcds = 8;

constexpr int kMinWavesPerSimd = 2;   // register budget of both tile shapes: 256 VGPRs per lane


template <int BM_, int BN_, int BK_, int WM_, int WN_, bool EARLY_ = false, int KG_ = 1>
struct Cfg {
    // KG: wave groups per block.  Each group computes the whole BM x BN tile over its own KSLICE-wide
    // slice of every k tile (the block stages KG slices at a time), and the groups' accumulators are
    // added in group order through LDS at the end: more waves per SIMD on a tile too small to give
    // each its own piece of C, without a second launch to add the parts.
    static constexpr int BM = BM_, BN = BN_, KSLICE = BK_, KG = KG_, BK = BK_ * KG_, WM = WM_, WN = WN_;
    // EARLY: the staged tile goes to LDS, and the next tile is requested from global memory, at the
    // top of a k tile instead of around its barrier.  The request then has a whole k tile to arrive;
    // where a k tile is a handful of MFMAs (the 64 x 64 and 128 x 128 block tiles: 8 and 32 per wave)
    // the later place left it half of that, less than the latency of the L2.
    static constexpr bool EARLY = EARLY_;
    static constexpr int TM = WM / 32, TN = WN / 32;       // MFMA tiles per wave
    static constexpr int WAVES_N = BN / WN;
    static constexpr int WAVES_MN = (BM / WM) * (BN / WN);
    static constexpr int THREADS = WAVES_MN * KG * 64;
    static_assert(THREADS == 256 || THREADS == 512 || THREADS == 1024, "4, 8 or 16 waves per block");
    static_assert(KSLICE % 8 == 0, "a group's k slice is a multiple of the 8-wide chunk");
    static constexpr int KPAD = BK + 4;                    // K-contiguous row stride (floats)
    static constexpr int XPAD_M = BM + 8, XPAD_N = BN + 8; // X-contiguous row strides
};

// LDS footprint of one operand tile (floats)
template <class C, bool KC, bool IS_A>
constexpr int tile_floats() {
    return KC ? (IS_A ? C::BM : C::BN) * C::KPAD : C::BK * (IS_A ? C::XPAD_M : C::XPAD_N);
}

// Global -> registers for one operand tile.  ROWS x BK (K-contiguous) or BK x ROWS
// (X-contiguous), as 128-bit pieces dealt to the 256 threads.
template <int ROWS, int BK, bool KC, int THREADS>
struct Stage {
    static constexpr int PIECES = ROWS * BK / 4 / THREADS;
    static_assert(ROWS * BK / 4 % THREADS == 0, "tile must split evenly over the block");
    v4f r[PIECES];
    const char* base;           // interior tiles: block-uniform address of the tile's current k position
    unsigned off;               // this thread's byte offset of piece 0 from `base`
    unsigned piece_step;        // block-uniform byte distance between consecutive pieces of a thread

    // Interior tiles (whole tile inside the matrix, aligned rows): no bounds logic in the loop.  The
    // address of piece q is (uniform base + q * uniform step) + one 32-bit per-thread offset, which
    // the compiler turns into scalar-base + vector-offset loads: one address register per operand
    // and only scalar arithmetic per k tile.  Needs the tile's byte extent below 2^32.
    __device__ __forceinline__ void init_fast(const float* __restrict__ p, int64_t ld, int x0, int k0) {
        constexpr int PER = KC ? (BK / 4) : (ROWS / 4);          // 128-bit pieces per contiguous row
        const int outer = threadIdx.x / PER, inner = (threadIdx.x % PER) * 4;
        base = reinterpret_cast<const char*>(KC ? p + int64_t(x0) * ld + k0 : p + int64_t(k0) * ld + x0);
        off = unsigned((int64_t(outer) * ld + inner) * 4);
        static_assert(THREADS % PER == 0, "pieces of one thread are whole rows apart");
        piece_step = unsigned(int64_t(THREADS / PER) * ld * 4);
    }
    __device__ __forceinline__ void load_fast(int64_t step_bytes) {
#pragma unroll
        for (int q = 0; q < PIECES; ++q)
            r[q] = *reinterpret_cast<const v4f*>(base + size_t(q) * piece_step + off);
        base += step_bytes;
    }
    // x0: first row/col of the tile in the X dimension, k0: first k; dimX, K: extents; ld: leading
    // dimension (elements) of the contiguous direction's rows.  VEC: 16-byte aligned rows.
    template <bool VEC>
    __device__ __forceinline__ void load(const float* __restrict__ p, int64_t ld, int x0, int k0, int dimX, int k_end) {
#pragma unroll
        for (int q = 0; q < PIECES; ++q) {
            int idx = threadIdx.x + q * THREADS;
            int outer, inner;   // outer indexes rows of the contiguous direction
            if (KC) { outer = idx / (BK / 4); inner = (idx % (BK / 4)) * 4; }
            else { outer = idx / (ROWS / 4); inner = (idx % (ROWS / 4)) * 4; }
            int gx = KC ? x0 + outer : x0 + inner;          // position along X
            int gk = KC ? k0 + inner : k0 + outer;          // position along K
            const float* src = KC ? p + int64_t(gx) * ld + gk : p + int64_t(gk) * ld + gx;
            int lim_outer = KC ? dimX : k_end, pos_outer = KC ? gx : gk;
            int lim_inner = KC ? k_end : dimX, pos_inner = KC ? gk : gx;
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (pos_outer < lim_outer) {
                if (VEC && pos_inner + 4 <= lim_inner) {
                    v = *reinterpret_cast<const v4f*>(src);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (pos_inner + e < lim_inner) v[e] = src[e];
                }
            }
            r[q] = v;
        }
    }
    __device__ __forceinline__ void store(float* __restrict__ lds, int stride) const {
#pragma unroll
        for (int q = 0; q < PIECES; ++q) {
            int idx = threadIdx.x + q * THREADS;
            int outer, inner;
            if (KC) { outer = idx / (BK / 4); inner = (idx % (BK / 4)) * 4; }
            else { outer = idx / (ROWS / 4); inner = (idx % (ROWS / 4)) * 4; }
            *reinterpret_cast<v4f*>(lds + outer * stride + inner) = r[q];
        }
    }
};

// Fragment fetch for one 32-wide MFMA tile and one 8-wide k chunk: f[s] is this lane's operand
// for k = chunk*8 + 4*(lane/32) + s.
template <bool KC>
__device__ __forceinline__ void fetch(const float* __restrict__ lds, int stride, int x, int kbase, float (&f)[4]) {
    if (KC) {
        v4f v = *reinterpret_cast<const v4f*>(lds + x * stride + kbase);
#pragma unroll
        for (int s = 0; s < 4; ++s) f[s] = v[s];
    } else {
#pragma unroll
        for (int s = 0; s < 4; ++s) f[s] = lds[(kbase + s) * stride + x];
    }
}

struct GemmArgs {
    const float* a; int64_t lda;
    const float* b; int64_t ldb;
    float* c; int64_t ldc;          // C
    int m, n, k;
    int tiles_m, tiles_n;
    // Tiles [0, whole_tiles) are computed by one block each over all of K.  The remaining tiles - the
    // last, partly filled round of blocks - are cut along K into `splits` parts of k_per_split, one
    // block each: block whole_tiles + (t - whole_tiles) * splits + z computes part z of tile t.
    int whole_tiles;
    int splits;
    int k_per_split;                // multiple of BK
    float* partial;                 // [split tiles][splits][BM][BN]
    int c_vec;                      // rows of C are 16-byte aligned
    const float* bias;              // optional row vector [n] added to every row of C (null: none)
    int relu;                       // then max(0, .) when set
    const float* mask;              // optional [m, n] row-major: C is multiplied by [mask > 0] last (null: none)
    // The column sums of b ([k, n] in contiguous rows) riding along (sum_out null: not wanted): blocks
    // [product_blocks, product_blocks + sum.chunks) of the product's launch run stage 1 of the narrow
    // column sum into sum_partials, and the last blocks of the launch that adds the parts run stage 2.
    float* sum_out;
    float* sum_partials;
    ColsumNarrowPlan sum;
    int product_blocks;
};

// Output epilogue of a product that is not split along K: bias add, then ReLU as `v > 0 ? v : +0`
// (NaN -> 0, -0 -> +0), each rounded as the separate Add and ReLU kernels round them, so that the
// fused product equals the three launches bit for bit.
__device__ __forceinline__ float epilogue(float v, const float* __restrict__ bias, int col, int relu) {
    if (bias) v = v + bias[col];
    if (relu) v = v > 0.0f ? v : 0.0f;
    return v;
}
// The gradient of a ReLU applied to a product that has just been formed: v * [y > 0] with the 0 / 1
// factor the separate kernel multiplies by (a zero keeps v's sign, NaN and infinities give NaN).
__device__ __forceinline__ float masked(float v, const float* __restrict__ mask, int64_t at) {
    return mask ? v * (mask[at] > 0.0f ? 1.0f : 0.0f) : v;
}

// One k tile of the pipelined loop and of the bounds-checked loop, as text: both start from tile t in LDS,
// tile t+1 in the staging registers and chunk 0 of tile t fetched, and leave the same for t+1.  (Text, not a
// lambda: the loop of the whole-K products must compile exactly as if the hand-over below did not exist.)
// In the pipelined tile with EARLY the buffer cur ^ 1 is free since the last barrier and its first readers
// wait behind the next, so the staged tile goes to LDS and the next is requested at the top.
#define CTAMD_PIPELINED_TILE(t) \
    {   \
            const int cur = t & 1; \
            __builtin_amdgcn_sched_barrier(0); \
            if (C::EARLY) { \
                sa.store(s_a[cur ^ 1], A_STRIDE); \
                sb.store(s_b[cur ^ 1], B_STRIDE); \
                const bool more = t + 3 < ktiles; \
                sa.load_fast(more ? a_step : 0); \
                sb.load_fast(more ? b_step : 0); \
                __builtin_amdgcn_sched_barrier(0); \
            } \
            lds_wait(); \
            fetch_chunk(cur, 1, 1); \
            mfmas(0); \
            if (!C::EARLY) { \
                sa.store(s_a[cur ^ 1], A_STRIDE); \
                sb.store(s_b[cur ^ 1], B_STRIDE); \
            } \
    _Pragma("unroll") \
            for (int q = 0; q < kReadSlots; ++q) { \
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 0); \
                __builtin_amdgcn_sched_group_barrier(kMaskDsRead, 1, 0); \
            } \
            if (C::EARLY) { \
                if (kMfmaPerChunk - kReadSlots > 0) __builtin_amdgcn_sched_group_barrier(kMaskMfma, kMfmaPerChunk - kReadSlots, 0); \
            } else { \
                if (kMfmaPerChunk - kReadSlots - kStores > 0) \
                    __builtin_amdgcn_sched_group_barrier(kMaskMfma, kMfmaPerChunk - kReadSlots - kStores, 0); \
    _Pragma("unroll") \
                for (int q = 0; q < kStores; ++q) { \
                    __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 0); \
                    __builtin_amdgcn_sched_group_barrier(kMaskDsWrite, 1, 0); \
                } \
            } \
            __builtin_amdgcn_sched_barrier(0); \
            __syncthreads(); \
            __builtin_amdgcn_sched_barrier(0); \
            fetch_chunk(cur ^ 1, 0, 0); \
            if (!C::EARLY) { \
                const bool more = t + 3 < ktiles; \
                sa.load_fast(more ? a_step : 0); \
                sb.load_fast(more ? b_step : 0); \
            } \
            mfmas(1); \
    _Pragma("unroll") \
            for (int q = 0; q < kReadSlots; ++q) { \
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 1); \
                __builtin_amdgcn_sched_group_barrier(kMaskDsRead, 1, 1); \
            } \
            if (C::EARLY) { \
                if (kMfmaPerChunk - kReadSlots > 0) __builtin_amdgcn_sched_group_barrier(kMaskMfma, kMfmaPerChunk - kReadSlots, 1); \
            } else { \
    _Pragma("unroll") \
                for (int q = 0; q < kStores; ++q) { \
                    __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 1); \
                    __builtin_amdgcn_sched_group_barrier(kMaskVmemRead, 1, 1); \
                } \
                if (kMfmaPerChunk - kReadSlots - kStores > 0) \
                    __builtin_amdgcn_sched_group_barrier(kMaskMfma, kMfmaPerChunk - kReadSlots - kStores, 1); \
            } \
            __builtin_amdgcn_sched_barrier(0); \
    }
#define CTAMD_CHECKED_TILE(t) \
    {   \
            const int cur = t & 1; \
            lds_wait(); \
            fetch_chunk(cur, 1, 1); \
            __builtin_amdgcn_sched_barrier(0); \
            mfmas(0); \
            __builtin_amdgcn_sched_barrier(0); \
            sa.store(s_a[cur ^ 1], A_STRIDE); \
            sb.store(s_b[cur ^ 1], B_STRIDE); \
            __syncthreads(); \
            fetch_chunk(cur ^ 1, 0, 0); \
            if (t + 2 < ktiles) stage_tile(t + 2); \
            __builtin_amdgcn_sched_barrier(0); \
            mfmas(1); \
            __builtin_amdgcn_sched_barrier(0); \
    }
// RAGGED: the launch's K is no whole number of k tiles (and rows are aligned): blocks inside C keep the
// pipelined loop for their whole k tiles and finish on the bounds-checked one.  A kernel of its own
// because the hand-over, merely by being there, cost the loop of the whole-K products 0.9% (registers
// and address arithmetic around the same 64 MFMAs: 4096^3 955 -> 962 us).
template <class C, bool A_KC, bool B_KC, bool VEC, bool SUMS = false, bool RAGGED = false>
__global__ __launch_bounds__(C::THREADS, kMinWavesPerSimd) void gemm_kernel(GemmArgs g) {
    constexpr int BM = C::BM, BN = C::BN, BK = C::BK, TM = C::TM, TN = C::TN;
    constexpr int A_STRIDE = A_KC ? C::KPAD : C::XPAD_M;
    constexpr int B_STRIDE = B_KC ? C::KPAD : C::XPAD_N;
    constexpr int A_FLOATS = tile_floats<C, A_KC, true>();
    constexpr int B_FLOATS = tile_floats<C, B_KC, false>();
    __shared__ __attribute__((aligned(16))) float s_a[2][A_FLOATS];
    __shared__ __attribute__((aligned(16))) float s_b[2][B_FLOATS];
    constexpr int KG = C::KG;
    __shared__ __attribute__((aligned(16))) float s_sum[KG > 1 ? (KG - 1) * BM * BN : 4];   // the other groups' accumulators

    if (SUMS && int(blockIdx.x) >= g.product_blocks) {
        static_assert(!SUMS || (2 * A_FLOATS >= kColsumThreads * 4 && !B_KC && VEC), "stage 1 borrows the A tiles' LDS; b in aligned contiguous rows");
        colsum_narrow_body<true>(g.b, g.sum_partials, size_t(g.k), size_t(g.n), g.sum.lanes, g.sum.groups, g.sum.rows_per_block,
                                 blockIdx.x - unsigned(g.product_blocks), threadIdx.x, &s_a[0][0]);
        return;
    }
    // XCD-aware renumbering: hardware block b runs on XCD b % 8; give each XCD a contiguous run of
    // tiles, and inside the run walk C in column-major bands of 8 tile rows so that co-resident
    // blocks share A row bands and B column bands in that XCD's L2.
    int bid = blockIdx.x, part = 0;
    const bool split = bid >= g.whole_tiles;
    if (!split) {
        int per = g.whole_tiles / kXcds, rem = g.whole_tiles % kXcds;
        int xcd = bid % kXcds, local = bid / kXcds;
        // XCDs with index < rem own per+1 tiles
        bid = xcd * per + (xcd < rem ? xcd : rem) + local;
    } else {
        const int r = bid - g.whole_tiles;
        bid = g.whole_tiles + r / g.splits;
        part = r % g.splits;
    }
    constexpr int BAND = 8;
    int band = bid / (BAND * g.tiles_n);
    int band_rows = g.tiles_m - band * BAND < BAND ? g.tiles_m - band * BAND : BAND;
    int in_band = bid - band * BAND * g.tiles_n;
    const int tile_m = band * BAND + in_band % band_rows;
    const int tile_n = in_band / band_rows;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int k_begin = split ? part * g.k_per_split : 0;
    int k_end = split ? k_begin + g.k_per_split : g.k;
    if (k_end > g.k) k_end = g.k;

    const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) % C::WAVES_MN, group = (threadIdx.x >> 6) / C::WAVES_MN;
    const int wm = (wave / C::WAVES_N) * C::WM, wn = (wave % C::WAVES_N) * C::WN;
    const int l32 = lane & 31, half = lane >> 5;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    Stage<BM, BK, A_KC, C::THREADS> sa;
    Stage<BN, BK, B_KC, C::THREADS> sb;
    const int ktiles = (k_end - k_begin + BK - 1) / BK;
    // interior: the whole BM x BN tile lies inside C, rows are 16-byte aligned and K is a whole number of k
    // tiles (RAGGED: at least two whole ones) - true for all blocks of a 4096^3 product, false only on ragged edges
    const bool interior = VEC && m0 + BM <= g.m && n0 + BN <= g.n &&
                          (RAGGED ? ((k_end - k_begin) % BK == 0 || (k_end - k_begin) / BK >= 2) : (k_end - k_begin) % BK == 0) &&
                          g.lda < (int64_t(1) << 21) && g.ldb < (int64_t(1) << 21);   // tile extent < 2^32 bytes
    const int64_t a_step = (A_KC ? BK : int64_t(BK) * g.lda) * 4;   // bytes per k tile
    const int64_t b_step = (B_KC ? BK : int64_t(BK) * g.ldb) * 4;
    if (interior) {
        sa.init_fast(g.a, g.lda, m0, k_begin);
        sb.init_fast(g.b, g.ldb, n0, k_begin);
    }
    // s_waitcnt lgkmcnt(0) as an instruction the compiler's wait-count bookkeeping sees (it cannot
    // look inside inline asm): vmcnt and expcnt fields at their maxima, lgkmcnt 0.
    auto lds_wait = [] { __builtin_amdgcn_s_waitcnt(0xC07F); };
    constexpr int NCH = C::KSLICE / 8;
    static_assert(NCH == 2, "the pipeline below alternates two fragment buffers over two chunks");
    float fa[2][TM][4], fb[2][TN][4];
    auto fetch_chunk = [&](int buf, int ch, int which) {
        const float* __restrict__ la = s_a[buf];
        const float* __restrict__ lb = s_b[buf];
        const int kb = group * C::KSLICE + ch * 8 + half * 4;
#pragma unroll
        for (int i = 0; i < TM; ++i) fetch<A_KC>(la, A_STRIDE, wm + i * 32 + l32, kb, fa[which][i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) fetch<B_KC>(lb, B_STRIDE, wn + j * 32 + l32, kb, fb[which][j]);
    };
    auto mfmas = [&](int which) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[which][i][s], fb[which][j][s], acc[i][j], 0, 0, 0);
    };
    constexpr int kMfmaPerChunk = 4 * TM * TN;
    constexpr int kStores = Stage<BM, BK, A_KC, C::THREADS>::PIECES + Stage<BN, BK, B_KC, C::THREADS>::PIECES;
    static_assert(kMfmaPerChunk >= 2 * kStores, "a burst has room for the tile's LDS stores and global loads");
    // LDS reads of one chunk: at most 4 per MFMA tile of an operand (32-bit reads of the
    // X-contiguous kind, which the compiler pairs up) - slots for them, one after each leading MFMA
    constexpr int kReadSlots = (2 * (TM + TN) < kMfmaPerChunk - kStores) ? 2 * (TM + TN) : kMfmaPerChunk - kStores;
    constexpr int kMaskMfma = 0x008, kMaskVmemRead = 0x020, kMaskDsRead = 0x100, kMaskDsWrite = 0x200;

    // Software pipeline over the two 8-wide k chunks of a k tile, two fragment buffers:
    //   burst 0: MFMAs of chunk 0 | issued under them: LDS reads of chunk 1, and at the tail the
    //            staged tile t+1 registers -> LDS;                      then the tile's one barrier
    //   burst 1: MFMAs of chunk 1 | issued under them: LDS reads of chunk 0 of tile t+1 and the
    //            global loads of tile t+2
    // so every fragment is requested most of a burst before its first use and a global load has a
    // whole k tile to arrive.  A wave issues in order, and an MFMA keeps the matrix pipe busy for
    // 64 cycles, so one memory instruction slipped in after an MFMA is free; what must not happen
    // is a wait in front of an MFMA for data requested just before it.  Interior blocks pin the
    // interleaving with scheduling groups; the two waves of a SIMD run in phase (one barrier per
    // tile), so housekeeping outside the bursts would idle the pipe for both.
    const int64_t span_k = k_end - k_begin;
    if constexpr (!RAGGED) {
        if (interior) {
            sa.load_fast(a_step);
            sb.load_fast(b_step);
            sa.store(s_a[0], A_STRIDE);
            sb.store(s_b[0], B_STRIDE);
            __syncthreads();
            // the loop always requests tile t+2; past the end the request repeats the last tile
            // (in bounds, never stored), which keeps the loop body free of branches
            if (ktiles > 1) { sa.load_fast(ktiles > 2 ? a_step : 0); sb.load_fast(ktiles > 2 ? b_step : 0); }
            fetch_chunk(0, 0, 0);
            for (int t = 0; t + 1 < ktiles; ++t) CTAMD_PIPELINED_TILE(t)
        } else {
            auto stage_tile = [&](int kt) {
                sa.template load<VEC>(g.a, g.lda, m0, k_begin + kt * BK, g.m, k_end);
                sb.template load<VEC>(g.b, g.ldb, n0, k_begin + kt * BK, g.n, k_end);
            };
            stage_tile(0);
            sa.store(s_a[0], A_STRIDE);
            sb.store(s_b[0], B_STRIDE);
            __syncthreads();
            if (ktiles > 1) stage_tile(1);
            fetch_chunk(0, 0, 0);
            for (int t = 0; t + 1 < ktiles; ++t) CTAMD_CHECKED_TILE(t)
        }
    } else {
        auto stage_tile = [&](int kt) {
            sa.template load<VEC>(g.a, g.lda, m0, k_begin + kt * BK, g.m, k_end);
            sb.template load<VEC>(g.b, g.ldb, n0, k_begin + kt * BK, g.n, k_end);
        };
        int t = 0;
        if (interior) {
            sa.load_fast(a_step);
            sb.load_fast(b_step);
            sa.store(s_a[0], A_STRIDE);
            sb.store(s_b[0], B_STRIDE);
            __syncthreads();
            if (ktiles > 1) { sa.load_fast(ktiles > 2 ? a_step : 0); sb.load_fast(ktiles > 2 ? b_step : 0); }
            fetch_chunk(0, 0, 0);
            // the pipelined loop while the tile it requests, two ahead, is a whole one
            const int fast_iters = span_k % BK == 0 ? ktiles - 1 : int(span_k / BK) - 2;
            for (; t < fast_iters; ++t) CTAMD_PIPELINED_TILE(t)
        } else {
            stage_tile(0);
            sa.store(s_a[0], A_STRIDE);
            sb.store(s_b[0], B_STRIDE);
            __syncthreads();
            if (ktiles > 1) stage_tile(1);
            fetch_chunk(0, 0, 0);
        }
        for (; t + 1 < ktiles; ++t) CTAMD_CHECKED_TILE(t)
    }
    // last k tile: nothing left to stage
    {
        const int cur = (ktiles - 1) & 1;
        lds_wait();
        fetch_chunk(cur, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mfmas(0);
        __builtin_amdgcn_sched_barrier(0);
        lds_wait();
        mfmas(1);
    }

    if (KG > 1) {
        // group 0 adds the other groups' accumulators to its own in group order; lane-contiguous
        // words, so neither side meets a bank conflict
        float* __restrict__ mine = s_sum + (size_t(group > 0 ? group - 1 : 0) * C::WAVES_MN + wave) * (TM * TN * 16 * 64) + lane;
        if (group > 0) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mine[((i * TN + j) * 16 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (group > 0) return;
#pragma unroll
        for (int z = 1; z < KG; ++z)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[i][j][r] += mine[(size_t(z - 1) * C::WAVES_MN * TM * TN * 16 + (i * TN + j) * 16 + r) * 64];
    }
    // accumulator register r of lane l holds C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 tile
    if (!split) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = n0 + wn + j * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                    if (row < g.m && col < g.n)
                        g.c[int64_t(row) * g.ldc + col] = masked(epilogue(acc[i][j][r], g.bias, col, g.relu), g.mask, int64_t(row) * g.ldc + col);
                }
            }
        return;
    }
    // A part of a split tile: the partial product goes to this part's [BM][BN] buffer (whole, the
    // rows and columns past the edge of C are zeros); fold_parts adds the parts up.
    const int split_tile = bid - g.whole_tiles;
    float* __restrict__ mine = g.partial + (size_t(split_tile) * g.splits + part) * (BM * BN);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = wn + j * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = wm + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                mine[row * BN + col] = acc[i][j][r];
            }
        }
}

#undef CTAMD_PIPELINED_TILE
#undef CTAMD_CHECKED_TILE

// Adds the parts of the split tiles in their order and writes C (bias and ReLU of the fused
// product included): blockIdx.x is the split tile, blockIdx.y one of its slices of kFoldSlice elements.
constexpr int kFoldSlice = kThreads * 4;       // one 128-bit word per thread: a tile cut in many parts has few tiles, and the grid is tiles x slices
template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void fold_parts(GemmArgs g) {
    static_assert(BM * BN % kFoldSlice == 0, "a tile is a whole number of slices");
    __shared__ double s_acc[kColsumThreads];
    if (blockIdx.x >= unsigned(g.tiles_m * g.tiles_n - g.whole_tiles)) {       // past the split tiles: stage 2 of b's column sums
        if (blockIdx.y == 0)
            colsum_fold_body<kFoldLanes>(g.sum_partials, g.sum_out, size_t(g.n), g.sum.chunks,
                                         blockIdx.x - unsigned(g.tiles_m * g.tiles_n - g.whole_tiles), threadIdx.x, s_acc);
        return;
    }
    const int split_tile = blockIdx.x;
    const int bid = g.whole_tiles + split_tile;
    constexpr int BAND = 8;
    const int band = bid / (BAND * g.tiles_n);
    const int band_rows = g.tiles_m - band * BAND < BAND ? g.tiles_m - band * BAND : BAND;
    const int in_band = bid - band * BAND * g.tiles_n;
    const int m0 = (band * BAND + in_band % band_rows) * BM, n0 = (in_band / band_rows) * BN;
    const float* __restrict__ parts = g.partial + size_t(split_tile) * g.splits * (BM * BN);
    const int first = blockIdx.y * (kFoldSlice / 4);
    for (int idx = first + threadIdx.x; idx < first + kFoldSlice / 4; idx += kThreads) {
        const int row = idx / (BN / 4), col = (idx % (BN / 4)) * 4;
        const int grow = m0 + row, gcol = n0 + col;
        if (grow >= g.m || gcol >= g.n) continue;
        const v4f* __restrict__ src = reinterpret_cast<const v4f*>(parts + row * BN + col);
        constexpr size_t kStep = size_t(BM) * BN / 4;      // 128-bit words between parts
        v4f t = src[0];
        int z = 1;
        for (; z + 7 < g.splits; z += 8) {     // eight loads in flight, added in order of z
            v4f p[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) p[q] = src[size_t(z + q) * kStep];
#pragma unroll
            for (int q = 0; q < 8; ++q) t = t + p[q];
        }
        for (; z < g.splits; ++z) t = t + src[size_t(z) * kStep];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (gcol + e < g.n) t[e] = masked(epilogue(t[e], g.bias, gcol + e, g.relu), g.mask, int64_t(grow) * g.ldc + gcol + e);
        float* __restrict__ dst = g.c + int64_t(grow) * g.ldc + gcol;
        if (g.c_vec && gcol + 4 <= g.n) {
            *reinterpret_cast<v4f*>(dst) = t;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (gcol + e < g.n) dst[e] = t[e];
        }
    }
}

// ---- Small products: at most one 32 x 32 tile of C per CU.  The big tiles put such a product on a
// handful of CUs, where it runs at those CUs' MFMA rate, or cut K over blocks and pay a second
// launch to add the parts.  Here a block owns one 32 x 32 tile and its 16 waves share out K in
// runs of 32-wide spans: every wave feeds its MFMA operands straight from global memory - lane l
// holds row / column l % 32 at the 16 consecutive k of its half of the span (the sum over k is
// order-free, so both operands simply use the same labelling; an operand contiguous in k is read
// 64 bytes per lane) - with one span being multiplied while the next is on its way, and the 16
// accumulator tiles are added in order through LDS.
constexpr int kMicroWaves = 16;
constexpr int kMicroSpan = 32;
constexpr int kMicroMaxK = 512;
struct MicroArgs {
    const float* a; int64_t lda;       // lda, ldb: as in GemmArgs
    const float* b; int64_t ldb;
    float* c;
    int m, n, k, tiles_m;
    int spans_per_wave;
    const float* bias; int relu;
    const float* mask;                 // as in GemmArgs
    // the column sums of a small contiguous matrix, carried along as the blocks after the `tiles` of
    // the product (sum_out null: none): the bias gradient of a layer beside its weight gradient
    int tiles;
    const float* sum_src; float* sum_out;
    size_t sum_cols; unsigned sum_rows;
};
// f[i] = operand element (x, k0 + i), i < 16; zeros past k or when x is outside the matrix
template <bool KC, bool VEC>
__device__ __forceinline__ void micro_fetch(const float* __restrict__ p, int64_t ld, int x, bool x_ok, int k0, int k, float (&f)[16]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] = 0.0f;
    if (!x_ok) return;
    if (KC) {
        const float* __restrict__ src = p + int64_t(x) * ld + k0;
        if (VEC && k0 + 16 <= k) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4f v = reinterpret_cast<const v4f*>(src)[q];
#pragma unroll
                for (int e = 0; e < 4; ++e) f[4 * q + e] = v[e];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (k0 + i < k) f[i] = src[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            if (k0 + i < k) f[i] = p[int64_t(k0 + i) * ld + x];
    }
}
template <bool A_KC, bool B_KC, bool VEC>
__global__ __launch_bounds__(kMicroWaves * 64) void gemm_micro(MicroArgs g) {
    __shared__ float s_red[kMicroWaves * 16 * 64];
    if (blockIdx.x >= unsigned(g.tiles)) {         // block-uniform: one of the column-sum blocks
        static_assert(sizeof(s_red) >= kColsumThreads * sizeof(double), "the column sums borrow the product's LDS");
        colsum_fold_body<kSmallLanes>(g.sum_src, g.sum_out, g.sum_cols, g.sum_rows, blockIdx.x - unsigned(g.tiles), threadIdx.x,
                                      reinterpret_cast<double*>(s_red));
        return;
    }
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(int(threadIdx.x) >> 6);
    const int m0 = (blockIdx.x % g.tiles_m) * 32, n0 = (blockIdx.x / g.tiles_m) * 32;
    const int row = m0 + l32, col = n0 + l32;
    const bool row_ok = row < g.m, col_ok = col < g.n;
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    // this wave's spans: [first, last), wave-uniform
    const int spans = (g.k + kMicroSpan - 1) / kMicroSpan;
    const int first = wave * g.spans_per_wave;
    const int last = first + g.spans_per_wave < spans ? first + g.spans_per_wave : spans;
    float fa[2][16], fb[2][16];
    auto request = [&](int span, int buf) {
        const int k0 = span * kMicroSpan + 16 * half;
        micro_fetch<A_KC, VEC>(g.a, g.lda, row, row_ok, k0, g.k, fa[buf]);
        micro_fetch<B_KC, VEC>(g.b, g.ldb, col, col_ok, k0, g.k, fb[buf]);
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[buf][i], fb[buf][i], acc, 0, 0, 0);
    };
    if (first < last) request(first, 0);
    for (int sp = first; sp < last; sp += 2) {
        if (sp + 1 < last) request(sp + 1, 1);
        multiply(0);
        if (sp + 1 < last) {
            if (sp + 2 < last) request(sp + 2, 0);
            multiply(1);
        }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) s_red[(wave * 16 + r) * 64 + lane] = acc[r];
    __syncthreads();
    // value t = r * 64 + l is accumulator register r of lane l: C[8 (r / 4) + 4 (l / 32) + r % 4][l % 32]
    const int t = threadIdx.x, r = t >> 6, l = t & 63;
    float total = s_red[t];
#pragma unroll
    for (int w = 1; w < kMicroWaves; ++w) total = total + s_red[w * 1024 + t];
    const int crow = m0 + 8 * (r / 4) + 4 * (l / 32) + r % 4, ccol = n0 + (l & 31);
    if (crow < g.m && ccol < g.n)
        g.c[int64_t(crow) * g.n + ccol] = masked(epilogue(total, g.bias, ccol, g.relu), g.mask, int64_t(crow) * g.n + ccol);
}

template <bool A_KC, bool B_KC>
void launch_micro(const MicroArgs& g, bool vec, dim3 grid, dim3 block, hipStream_t s) {
    if (vec) hipLaunchKernelGGL((gemm_micro<A_KC, B_KC, true>), grid, block, 0, s, g);
    else hipLaunchKernelGGL((gemm_micro<A_KC, B_KC, false>), grid, block, 0, s, g);
}

// ---- Products with a narrow output, n <= 16: the logits of a classifier, [B x H] . [H x 10], and
// the gradient of its weights, [H x B] . [B x 10].  A 64 x 64 MFMA tile would compute 54 of its 64
// columns for nothing, and with rows of 10 floats B takes the element-wise edge path; these kernels
// stream A once on the vector units instead.  fp32 fused multiply-adds and sums in a fixed order:
// results are deterministic and the same for every row of the output.
constexpr int kNarrowN = 16;
constexpr int kNarrowRows = 4;                 // rows of A a wave works on at a time
constexpr int kNarrowLdsBytes = 64 << 10;

// Sums `P` values per lane over the 64 lanes of a wave in P + log2(64 / P) exchanges instead of
// 6 P: each step halves the values a lane still carries (the upper lanes of the pair keep the upper
// half).  Afterwards lane l holds the total of value l / (64 / P) in v[0].
template <int CNT, int OFF, int P>
__device__ __forceinline__ void wave_sums_step(float (&v)[P], int lane) {
    if constexpr (CNT > 1) {
        const bool upper = (lane & OFF) != 0;
#pragma unroll
        for (int j = 0; j < CNT / 2; ++j) {
            const float send = upper ? v[j] : v[j + CNT / 2];
            const float keep = upper ? v[j + CNT / 2] : v[j];
            v[j] = keep + __shfl_xor(send, OFF, 64);
        }
        wave_sums_step<CNT / 2, OFF / 2, P>(v, lane);
    } else if constexpr (OFF >= 1) {
        v[0] = v[0] + __shfl_xor(v[0], OFF, 64);
        wave_sums_step<1, OFF / 2, P>(v, lane);
    }
}
template <int P>
__device__ __forceinline__ void wave_sums(float (&v)[P], int lane) {
    static_assert(P >= 1 && P <= 64 && (P & (P - 1)) == 0, "a power of two");
    wave_sums_step<P, 32, P>(v, lane);
}
constexpr int pow2_at_least(int v) { return v <= 1 ? 1 : 2 * pow2_at_least((v + 1) / 2); }

// A K-contiguous (row-major [m, k]), B in rows of n.  B is staged transposed into LDS as [n][kp]
// (kp: k rounded up to the 256-wide slab, zeros behind k).  A wave takes kNarrowRows rows at a time:
// lane l holds A[row][k0 + 4l .. 4l + 3] of a slab and the 4 x n values of B those k meet, and the
// rows' n partial sums go round the wave.  VEC: rows of A are 16-byte aligned.  ONE_SLAB: k <= 256,
// B stays in registers for all rows and the next rows of A are requested while these are multiplied.
template <int N, bool VEC, bool ONE_SLAB>
__global__ __launch_bounds__(kThreads) void gemm_narrow_rows(const float* __restrict__ a, int64_t lda, const float* __restrict__ b,
                                                             int64_t ldb, float* __restrict__ c, int m, int k, int kp,
                                                             int turns, const float* __restrict__ bias, int relu) {
    extern __shared__ __attribute__((aligned(16))) float s_bt[];        // [N][kp]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int R = kNarrowRows;
    // the block's waves take consecutive groups of R rows, `turns` groups each, a block's rows in one run
    const int first = (blockIdx.x * (kThreads / 64) * turns + wave) * R;
    const int stride = (kThreads / 64) * R;
    auto load_rows = [&](int row0, int k0, v4f (&av)[R]) {
        const int kk = k0 + 4 * lane;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (row0 + r < m) {
                const float* src = a + int64_t(row0 + r) * lda + kk;
                if (VEC && kk + 4 <= k) v = *reinterpret_cast<const v4f*>(src);
                else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (kk + e < k) v[e] = src[e];
                }
            }
            av[r] = v;
        }
    };
    v4f av[R];
    if (ONE_SLAB) load_rows(first, 0, av);                     // on its way while B is staged
    for (int e = threadIdx.x; e < kp * N; e += kThreads) {
        const int l = e / N, q = e % N;
        s_bt[q * kp + l] = l < k ? b[int64_t(l) * ldb + q] : 0.0f;
    }
    __syncthreads();
    v4f bw[N];
    if (ONE_SLAB) {
#pragma unroll
        for (int q = 0; q < N; ++q) bw[q] = *reinterpret_cast<const v4f*>(s_bt + q * kp + 4 * lane);
    }
    constexpr int P = pow2_at_least(R * N);
    for (int t = 0; t < turns; ++t) {
        const int row0 = first + t * stride;
        if (row0 >= m) break;                                  // wave-uniform
        float acc[P];
#pragma unroll
        for (int v = 0; v < P; ++v) acc[v] = 0.0f;
        if (ONE_SLAB) {
            v4f next[R];
            if (t + 1 < turns) load_rows(row0 + stride, 0, next);
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int q = 0; q < N; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[r * N + q] = __fmaf_rn(av[r][e], bw[q][e], acc[r * N + q]);
            if (t + 1 < turns) {
#pragma unroll
                for (int r = 0; r < R; ++r) av[r] = next[r];
            }
        } else {
            for (int k0 = 0; k0 < k; k0 += 256) {
                load_rows(row0, k0, av);
#pragma unroll
                for (int q = 0; q < N; ++q) {
                    const v4f w = *reinterpret_cast<const v4f*>(s_bt + q * kp + k0 + 4 * lane);
#pragma unroll
                    for (int r = 0; r < R; ++r)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[r * N + q] = __fmaf_rn(av[r][e], w[e], acc[r * N + q]);
                }
            }
        }
        wave_sums<P>(acc, lane);
        constexpr int kLanesPerValue = 64 / P;
        const int v = lane / kLanesPerValue;
        if (lane % kLanesPerValue == 0 && v < R * N && row0 + v / N < m)
            c[int64_t(row0 + v / N) * N + v % N] = epilogue(acc[0], bias, v % N, relu);
    }
}

// A X-contiguous (the transposed view of a row-major [k, m]), B in rows of n.  A block of 16 waves
// owns 64 rows i of the output and a run of k; wave w takes l = w, w + 16, ... of the run, lane j
// reads A[l][i0 + j] (a wave reads 256 contiguous bytes, eight l in flight and the next eight
// requested) and multiplies it with B's row l, which all lanes read from LDS at one address.  The
// 16 waves' sums are added in order through the same LDS.  With the k range cut in several runs
// (gridDim.y) the results go to `out` as [run][m * n] and gemm_narrow_fold adds the runs.
constexpr int kNarrowWaves = 16;
template <int N>
__global__ __launch_bounds__(kNarrowWaves * 64) void gemm_narrow_cols(const float* __restrict__ a, int64_t lda,
                                                                      const float* __restrict__ b, int64_t ldb,
                                                                      float* __restrict__ out, int m, int k, int k_per_run,
                                                                      const float* __restrict__ bias, int relu) {
    constexpr int kChunk = kNarrowWaves * 64;                  // rows of B resident at a time
    __shared__ float s_mem[kChunk * N];                        // B's rows [kChunk][N]; at the end the sums [wave][N][64]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(int(threadIdx.x) >> 6);
    const int i = blockIdx.x * 64 + lane;
    const int k_begin = blockIdx.y * k_per_run;
    const int k_end = k_begin + k_per_run < k ? k_begin + k_per_run : k;
    constexpr int kAhead = 8, kStep = kNarrowWaves * kAhead;
    float acc[N];
#pragma unroll
    for (int q = 0; q < N; ++q) acc[q] = 0.0f;
    const bool mine = i < m;
    for (int c0 = k_begin; c0 < k_end; c0 += kChunk) {
        const int len = k_end - c0 < kChunk ? k_end - c0 : kChunk;
        const float* __restrict__ a0 = a + int64_t(c0) * lda + i;
        auto request = [&](int l0, float (&av)[kAhead]) {
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int l = l0 + u * kNarrowWaves;
                av[u] = (mine && l < len) ? a0[int64_t(l) * lda] : 0.0f;
            }
        };
        float av[kAhead];
        request(wave, av);                                     // on its way while B's rows are staged
        if (c0 != k_begin) __syncthreads();
        for (int e = threadIdx.x; e < len * N; e += kNarrowWaves * 64) s_mem[e] = b[int64_t(c0 + e / N) * ldb + e % N];
        __syncthreads();
        for (int l0 = wave; l0 < len; l0 += kStep) {
            float next[kAhead];
            if (l0 + kStep < len) request(l0 + kStep, next);
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int l = l0 + u * kNarrowWaves;
                if (l < len) {                                 // wave-uniform
#pragma unroll
                    for (int q = 0; q < N; ++q) acc[q] = __fmaf_rn(av[u], s_mem[l * N + q], acc[q]);
                }
            }
            if (l0 + kStep < len) {
#pragma unroll
                for (int u = 0; u < kAhead; ++u) av[u] = next[u];
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < N; ++q) s_mem[(wave * N + q) * 64 + lane] = acc[q];
    __syncthreads();
    const int t = threadIdx.x;
    if (t >= 64 * N) return;
    const int j = t / N, q = t % N;
    if (int(blockIdx.x) * 64 + j >= m) return;
    float total = s_mem[q * 64 + j];
#pragma unroll
    for (int w = 1; w < kNarrowWaves; ++w) total = total + s_mem[(w * N + q) * 64 + j];
    const size_t e = size_t(blockIdx.x) * 64 * N + t;          // = (i0 + j) * N + q
    if (gridDim.y > 1) out[size_t(blockIdx.y) * size_t(m) * N + e] = total;
    else out[e] = epilogue(total, bias, q, relu);
}
// 16 lanes per output element: lane j adds runs j, j + 16, ... in order, then the 16 go round.
template <int N>
__global__ __launch_bounds__(kThreads) void gemm_narrow_fold(const float* __restrict__ partial, float* __restrict__ c, int m, int runs,
                                                             const float* __restrict__ bias, int relu) {
    const size_t mn = size_t(m) * N;
    const size_t e = (size_t(blockIdx.x) * kThreads + threadIdx.x) / 16;
    const int j = threadIdx.x % 16;
    float t = 0.0f;
    if (e < mn) {
        for (int z = j; z < runs; z += 16 * 4) {
            float p[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) p[u] = z + 16 * u < runs ? partial[size_t(z + 16 * u) * mn + e] : 0.0f;
#pragma unroll
            for (int u = 0; u < 4; ++u) t = t + p[u];
        }
    }
#pragma unroll
    for (int off = 8; off >= 1; off /= 2) t = t + __shfl_xor(t, off, 64);
    if (e < mn && j == 0) c[e] = epilogue(t, bias, int(e % N), relu);
}

template <int N>
int launch_narrow(const char* name, bool rows_form, const float* a, int64_t lda, const float* b, int64_t ldb, const float* bias, int relu,
                  float* c, int m, int k, void* stream) {
    hipStream_t s = as_stream(stream);
    const int cus = compute_units() > 0 ? compute_units() : 256;
    if (rows_form) {
        const int kp = (k + 255) / 256 * 256;
        const int groups = (m + kNarrowRows - 1) / kNarrowRows;          // of kNarrowRows rows, one wave each
        const int waves = cus * (kThreads / 64);
        const int turns = (groups + waves - 1) / waves;
        const int blocks = (groups + turns * (kThreads / 64) - 1) / (turns * (kThreads / 64));
        const size_t lds = size_t(N) * kp * sizeof(float);
        const bool vec = aligned16(a) && lda % 4 == 0;
        auto kernel = k <= 256 ? (vec ? gemm_narrow_rows<N, true, true> : gemm_narrow_rows<N, false, true>)
                               : (vec ? gemm_narrow_rows<N, true, false> : gemm_narrow_rows<N, false, false>);
        hipLaunchKernelGGL(kernel, dim3(unsigned(blocks)), dim3(kThreads), lds, s, a, lda, b, ldb, c, m, k, kp, turns, bias, relu);
        return launched(name);
    }
    const int strips = (m + 63) / 64;
    // one run while a wave's share of k is short (a second launch costs more than it saves);
    // otherwise about one block per CU, and no run shorter than 128
    int runs = 1;
    if (k > 512) {
        runs = (cus + strips - 1) / strips;
        if (runs > k / 128) runs = k / 128;
        const size_t by_scratch = kScratchFloats / (size_t(m) * N);
        if (size_t(runs) > by_scratch) runs = int(by_scratch);
        if (runs < 1) runs = 1;
    }
    const int k_per_run = (k + runs - 1) / runs;
    runs = (k + k_per_run - 1) / k_per_run;
    ScratchUse use(stream, runs > 1);
    float* partial = use.ptr();
    if (runs > 1 && !partial) return CTAMD_EINVAL;
    hipLaunchKernelGGL(gemm_narrow_cols<N>, dim3(unsigned(strips), unsigned(runs)), dim3(kNarrowWaves * 64), 0, s, a, lda, b, ldb,
                       runs > 1 ? partial : c, m, k, k_per_run, bias, relu);
    int rc = launched(name);
    if (rc || runs == 1) return rc;
    hipLaunchKernelGGL(gemm_narrow_fold<N>, dim3(unsigned((size_t(m) * N * 16 + kThreads - 1) / kThreads)), dim3(kThreads), 0, s,
                       partial, c, m, runs, bias, relu);
    return launched(name);
}

// Operands with no unit stride: one thread per output element.  Correct for any strides; only
// the reference's own transposes of transposes could produce such views.
__global__ __launch_bounds__(kThreads) void gemm_strided(const float* __restrict__ a, int64_t as0, int64_t as1,
                                                         const float* __restrict__ b, int64_t bs0, int64_t bs1,
                                                         float* __restrict__ c, int m, int n, int k,
                                                         const float* __restrict__ bias, int relu) {
    size_t idx = size_t(blockIdx.x) * kThreads + threadIdx.x;
    if (idx >= size_t(m) * n) return;
    int i = int(idx / n), j = int(idx % n);
    float s = 0.0f;
    for (int l = 0; l < k; ++l) s = __fmaf_rn(a[i * as0 + l * as1], b[l * bs0 + j * bs1], s);
    c[idx] = epilogue(s, bias, j, relu);
}

// Four tile shapes; the host picks one, and a cut of the last round of tiles along K, by a model of
// the time each plan takes (matmul_impl).
//   Big   256 x 256 x 16, 8 waves of 128 x 64 (128 accumulator registers, two waves per SIMD): the
//         fewest LDS and global bytes per flop; 4096^3 in 0.95 ms (145 TFLOP/s), 8192^3 at 146.
//   Wide  256 x 128 x 16, 4 waves of 128 x 64, two blocks per CU: 1-5% behind Big per flop.
//   Small 128 x 128 x 16, 4 waves of 64 x 64, two blocks per CU: 7% behind Big per flop; with the 64
//         tiles that 3072^3 leaves after one round cut in four along K, 0.43 ms (134 TFLOP/s)
//         against 0.55 ms uncut.
//   Tiny  64 x 64 x 16, 4 waves of 32 x 32, up to 4 blocks per CU: 1024^3 in 28 us (76 TFLOP/s) and
//         the skinny products of a small layer ([8192 x 784] . [784 x 256] in 32 us), cut along K
//         when the tiles are fewer than the CUs ([784 x 8192] . [8192 x 256] in 43 us).
using BigTile = Cfg<256, 256, 16, 128, 64>;
using SmallTile = Cfg<128, 128, 16, 64, 64>;
using TinyTile = Cfg<64, 64, 16, 32, 32>;
using WideTile = Cfg<256, 128, 16, 128, 64>;
// the 64 x 64 tile for a launch of at most one block per CU: no other block hides the wait for the next
// tile ([1024 x 1024, K = 2048]: 67 -> 45 us; with several blocks per CU it is 1-2% slower, as is the
// 128 x 128 tile either way)
using TinyEarlyTile = Cfg<64, 64, 16, 32, 32, true>;
using TinyK4Tile = Cfg<64, 64, 16, 32, 32, true, 4>;
// the 128 x 128 tile for a launch of at most one block per CU: eight waves of 64 x 32 (2048^3: 129 / 133 us
// for A.B / A^T.B against 138 / 141 on the four-wave block and 131.5 / 135 on that block with two wave
// groups; [2048 x 2048, K = 256] 22.9 against 25.7 us), and for two K-contiguous operands with a long K
// sixteen: the same eight in two wave groups (A.B^T 2048^3 130.0 against 133.4 us)
using Small8Tile = Cfg<128, 128, 16, 64, 32, true>;
using Small16Tile = Cfg<128, 128, 16, 64, 32, false, 2>;
// the 256 x 256 tile as sixteen waves of 64 x 64, four per SIMD, for A.B^T and A^T.B: 4096^3 939 / 966 us
// against 956 / 976 on the eight-wave block, 8192^3 7.42 / 7.63 against 7.55 / 7.69 ms (A.B loses 4% on it)
using Big16Tile = Cfg<256, 256, 16, 64, 64, true>;

template <class Tile, bool A_KC, bool B_KC>
int launch_gemm(GemmArgs g, bool vec, int blocks, hipStream_t s) {
    const bool ragged = g.k % Tile::BK != 0;        // parts of a cut K are whole k tiles each, but for the last
    if (vec && ragged) hipLaunchKernelGGL((gemm_kernel<Tile, A_KC, B_KC, true, false, true>), dim3(unsigned(blocks)), dim3(Tile::THREADS), 0, s, g);
    else if (vec) hipLaunchKernelGGL((gemm_kernel<Tile, A_KC, B_KC, true>), dim3(unsigned(blocks)), dim3(Tile::THREADS), 0, s, g);
    else hipLaunchKernelGGL((gemm_kernel<Tile, A_KC, B_KC, false>), dim3(unsigned(blocks)), dim3(Tile::THREADS), 0, s, g);
    return launched("ctamd_matmul_f32");
}

// the product with stage 1 of b's column sums as extra blocks (b in contiguous aligned rows)
template <class Tile>
int launch_with_sums(GemmArgs g, bool a_kc, int blocks, hipStream_t s) {
    if (a_kc) hipLaunchKernelGGL((gemm_kernel<Tile, true, false, true, true>), dim3(unsigned(blocks)), dim3(Tile::THREADS), 0, s, g);
    else hipLaunchKernelGGL((gemm_kernel<Tile, false, false, true, true>), dim3(unsigned(blocks)), dim3(Tile::THREADS), 0, s, g);
    return launched("ctamd_matmul_colsum_f32");
}

template <class Tile>
int launch_layout(GemmArgs g, bool a_kc, bool b_kc, bool vec, int blocks, hipStream_t s) {
    if (a_kc && b_kc) return launch_gemm<Tile, true, true>(g, vec, blocks, s);
    if (a_kc) return launch_gemm<Tile, true, false>(g, vec, blocks, s);
    if (b_kc) return launch_gemm<Tile, false, true>(g, vec, blocks, s);
    return launch_gemm<Tile, false, false>(g, vec, blocks, s);
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

namespace {

// C = A.B, optionally followed by "+ bias row" and ReLU in the same launch (in the fold launch when
// the product is split along K).
// sums / sums_done (or null): the column sums of a contiguous b are wanted as well; *sums_done says
// whether the product's launch carried them (only the small-product kernel can).
int matmul_impl(const char* name, const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                const float* bias, int relu, const float* mask, float* c, int64_t m, int64_t n, int64_t k, void* stream,
                float* sums = nullptr, bool* sums_done = nullptr) {
    if (m < 0 || n < 0 || k < 0) return fail(CTAMD_EINVAL, "%s: negative extent", name);
    if (m == 0 || n == 0) return CTAMD_OK;
    if (!c) return fail(CTAMD_EINVAL, "%s: null output", name);
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff || m * n > (int64_t(1) << 40))
        return fail(CTAMD_ERANGE, "%s: extent too large", name);
    if (k == 0) {                                   // an empty sum: 0, then the epilogue
        int rc = ctamd_fill_f32(c, 0.0f, size_t(m) * size_t(n), stream);
        if (!rc && bias) rc = ctamd_add_rowbcast_f32(c, bias, c, size_t(m), size_t(n), stream);
        if (!rc && relu) rc = ctamd_relu_f32(c, c, size_t(m) * size_t(n), stream);
        if (!rc && mask) rc = ctamd_relu_backward_f32(mask, c, c, size_t(m) * size_t(n), stream);
        return rc;
    }
    if (!a || !b) return fail(CTAMD_EINVAL, "%s: null input", name);
    if (as0 < 0 || as1 < 0 || bs0 < 0 || bs1 < 0) return fail(CTAMD_EINVAL, "%s: negative stride", name);
    hipStream_t s = as_stream(stream);
    account(4.0 * (double(m) * double(k) + double(k) * double(n) + double(m) * double(n) + (bias ? double(n) : 0.0)),
            2.0 * double(m) * double(n) * double(k));

    // a one-row / one-column operand is contiguous in whichever direction has extent > 1
    const bool a_kc = (as1 == 1) || (k == 1 && as0 != 1), a_xc = (as0 == 1) || (m == 1);
    const bool b_xc = (bs1 == 1) || (n == 1 && bs0 != 1), b_kc = (bs0 == 1) || (k == 1);
    if (!(a_kc || a_xc) || !(b_kc || b_xc)) {
        hipLaunchKernelGGL(gemm_strided, dim3(unsigned((size_t(m) * n + kThreads - 1) / kThreads)), dim3(kThreads), 0, s,
                           a, as0, as1, b, bs0, bs1, c, int(m), int(n), int(k), bias, relu);
        int rc = launched(name);
        if (!rc && mask) rc = ctamd_relu_backward_f32(mask, c, c, size_t(m) * size_t(n), stream);   // in place, as its own launch
        return rc;
    }
    const bool A_KC = a_kc, B_KC = !b_xc;
    const int cus = compute_units() > 0 ? compute_units() : 256;
    {
        // one tile per CU at most, and a K a CU can stream by itself: a CU draws some tens of GB/s, and a
        // 32 x 32 tile needs 256 bytes per k - beyond a few hundred k the tiled plan's cut of K over
        // many CUs (and its second launch) is the faster way
        const int64_t tiles32 = ((m + 31) / 32) * ((n + 31) / 32);
        const bool use = tiles32 <= cus && k <= kMicroMaxK;
        if (use) {
            MicroArgs g;
            g.a = a; g.lda = A_KC ? as0 : as1;
            g.b = b; g.ldb = B_KC ? bs1 : bs0;
            g.c = c; g.m = int(m); g.n = int(n); g.k = int(k);
            g.tiles_m = int((m + 31) / 32);
            const int spans = int((k + kMicroSpan - 1) / kMicroSpan);
            g.spans_per_wave = (spans + kMicroWaves - 1) / kMicroWaves;
            g.bias = bias; g.relu = relu; g.mask = mask;
            g.tiles = int(tiles32);
            g.sum_src = nullptr; g.sum_out = nullptr; g.sum_cols = 0; g.sum_rows = 0;
            unsigned sum_blocks = 0;
            if (sums && sums_done && colsum_is_small(size_t(k), size_t(n))) {
                g.sum_src = b; g.sum_out = sums; g.sum_cols = size_t(n); g.sum_rows = unsigned(k);
                sum_blocks = colsum_small_blocks(size_t(n));
                *sums_done = true;
                account(4.0 * double(k) * double(n), double(k) * double(n), true);
            }
            const bool vec = (!A_KC || (aligned16(a) && g.lda % 4 == 0)) && (!B_KC || (aligned16(b) && g.ldb % 4 == 0));
            const dim3 grid{unsigned(tiles32) + sum_blocks}, block{unsigned(kMicroWaves * 64)};
            if (A_KC && B_KC) launch_micro<true, true>(g, vec, grid, block, s);
            else if (A_KC) launch_micro<true, false>(g, vec, grid, block, s);
            else if (B_KC) launch_micro<false, true>(g, vec, grid, block, s);
            else launch_micro<false, false>(g, vec, grid, block, s);
            return launched(name);
        }
    }
    // a narrow output from a B in rows of n: the streaming kernels
    if (n <= kNarrowN && bs1 == 1 && m < (int64_t(1) << 27)) {
        const bool rows_form = (as1 == 1 || k == 1) && size_t(n) * size_t((k + 255) / 256 * 256) * sizeof(float) <= size_t(kNarrowLdsBytes);
        const bool cols_form = as0 == 1 && as1 != 1;
        if (rows_form || cols_form) {
            const int64_t lda = rows_form ? as0 : as1;
            int rc = CTAMD_OK;
            switch (n) {
#define CTAMD_NARROW(N_) case N_: rc = launch_narrow<N_>(name, rows_form, a, lda, b, bs0, bias, relu, c, int(m), int(k), stream); break;
                CTAMD_NARROW(1) CTAMD_NARROW(2) CTAMD_NARROW(3) CTAMD_NARROW(4) CTAMD_NARROW(5) CTAMD_NARROW(6) CTAMD_NARROW(7) CTAMD_NARROW(8)
                CTAMD_NARROW(9) CTAMD_NARROW(10) CTAMD_NARROW(11) CTAMD_NARROW(12) CTAMD_NARROW(13) CTAMD_NARROW(14) CTAMD_NARROW(15) CTAMD_NARROW(16)
#undef CTAMD_NARROW
                default: break;
            }
            if (!rc && mask) rc = ctamd_relu_backward_f32(mask, c, c, size_t(m) * size_t(n), stream);   // in place, as its own launch
            return rc;
        }
    }
    constexpr int BK = 16;
    static_assert(BigTile::BK == 16 && WideTile::BK == 16 && SmallTile::BK == 16 && TinyTile::BK == 16, "all tile shapes step K alike");
    // The plan: a tile shape, and into how many parts along K the tiles of the last, partly filled
    // round of blocks are cut (a round: `together` resident blocks on each CU), by a model of the
    // time in seconds, fitted to measurements on this chip (1024^3 ... 7168^3 and the skinny
    // products of a small layer):
    //   a full round       together * per_flop * BM * BN * t    t = 2 k flops at one CU's peak rate
    //   the last round     c blocks on the busiest CU, each 1 / parts of a tile: one block alone runs
    //                      at `alone` (one wave per SIMD leaves the matrix pipe idle between k tiles),
    //                      `together` of them at together * per_flop, in between in proportion; plus
    //                      the memory latencies a block waits out before its first and after its last k tile
    //   adding the parts   a launch and the parts' bytes written and read once
    // parts fill the free places of the round with at least 8 k tiles each (4 when K allows no more).
    // A launch of at most one block per CU runs on kernels made for that: the 64 x 64 tile with four wave
    // groups per block when each block has a long enough run of K (1024^3 26 -> 24 us, [1024 x 1024,
    // K = 4096] 88 -> 76 us), the 128 x 128 tile as eight waves of 64 x 32, in two wave groups for two
    // K-contiguous operands with a long K (2048^3 138 - 141 -> 129 - 133 us; 153 us on four 64 x 64 tiles
    // per CU, which the old figure for a lone 128 x 128 block preferred).
    auto wave_groups = [&](int sh, int64_t blocks, int parts) -> int {
        if (blocks > cus || sh > 1) return 1;
        const int64_t run = (k + parts - 1) / parts;
        if (sh == 0) return run >= 512 ? 4 : 1;
        return (A_KC && B_KC && run >= 1024) ? 2 : 1;
    };
    struct Shape { int bm, bn, together; double per_flop, alone; };
    static const Shape shapes[4] = {{TinyTile::BM, TinyTile::BN, 4, 1.30, 1.70}, {SmallTile::BM, SmallTile::BN, 2, 1.07, 1.34},
                                    {BigTile::BM, BigTile::BN, 1, 1.00, 1.00}, {WideTile::BM, WideTile::BN, 2, 1.04, 1.32}};
    const double t_elem = 2.0 * double(k) / (157.3e12 * 0.92 / cus);
    int shape = 0, splits = 1, whole_tiles = 0, groups = 1;
    double best = -1.0;
    for (int sh = 0; sh < 4; ++sh) {
        const Shape& q = shapes[sh];
        const int64_t tiles = ((m + q.bm - 1) / q.bm) * ((n + q.bn - 1) / q.bn);
        const int64_t places = int64_t(cus) * q.together;
        const int64_t rounds = tiles / places, left = tiles % places;
        const double area = double(q.bm) * q.bn;
        int most = 1;
        if (left > 0) {
            int64_t want = places / left;
            const int64_t by_scratch = int64_t(kScratchFloats) / (left * q.bm * q.bn);
            if (want > by_scratch) want = by_scratch;
            for (int min_ktiles = 8; min_ktiles >= 4 && most == 1; min_ktiles /= 2) {
                const int64_t by_k = k / (min_ktiles * BK);
                const int64_t p = want < by_k ? want : by_k;
                if (p >= 2) most = int(p);
            }
        }
        // also: as many parts as keep the launch at one block per CU
        const int fit = rounds == 0 && left > 0 && cus / left < most ? int(cus / left) : 0;
        for (int parts : {1, fit, most / 2, most}) {
            if (parts < 1 || (parts == 1 && most > 1 && left == 0)) continue;
            double cost = double(rounds) * q.together * q.per_flop * area * t_elem;
            int kg = 1;
            if (left > 0) {
                const int64_t c = (left * parts + cus - 1) / cus;
                kg = rounds == 0 ? wave_groups(sh, left * parts, parts) : 1;
                const bool one_per_cu = rounds == 0 && left * parts <= cus;
                // (fitted at [2048 x 2048]: 8.7 us + 60 us per 1024 of K for the uncut eight-wave block; a cut
                // one keeps the four-wave block's figure, which its measured times are nearer to)
                const double alone = sh == 0 ? (kg == 4 ? 1.32 : q.alone) : (sh == 1 && one_per_cu && parts == 1) ? 1.08 : q.alone;
                const double busy = q.together == 1 ? alone
                                                    : alone + double(c - 1) * (q.together * q.per_flop - alone) / (q.together - 1);
                cost += busy * area * t_elem / parts + (rounds == 0 ? 3e-6 : 1e-6);
                if (parts > 1) cost += 6e-6 + double(left) * parts * area * 8.0 / 4e12;
            }
            if (best < 0.0 || cost < best) {
                best = cost; shape = sh; splits = parts; whole_tiles = int(parts > 1 ? tiles - left : tiles); groups = kg;
            }
        }
    }
    const int BM = shapes[shape].bm, BN = shapes[shape].bn;
    GemmArgs g;
    g.a = a; g.lda = A_KC ? as0 : as1;
    g.b = b; g.ldb = B_KC ? bs1 : bs0;
    g.c = c; g.ldc = n;
    g.m = int(m); g.n = int(n); g.k = int(k);
    g.tiles_m = int((m + BM - 1) / BM);
    g.tiles_n = int((n + BN - 1) / BN);
    g.bias = bias; g.relu = relu; g.mask = mask;
    g.sum_out = nullptr; g.sum_partials = nullptr; g.sum = ColsumNarrowPlan{0, 0, 0, 0}; g.product_blocks = 0;
    g.c_vec = (aligned16(c) && n % 4 == 0) ? 1 : 0;
    const bool vec = aligned16(a) && aligned16(b) && (g.lda % 4 == 0) && (g.ldb % 4 == 0);
    const int tiles = g.tiles_m * g.tiles_n;
    g.whole_tiles = whole_tiles;
    g.splits = splits;
    g.partial = nullptr;
    g.k_per_split = int(k);
    ScratchUse use(stream, splits > 1);
    if (splits > 1) {
        int kps = int((k + splits - 1) / splits);
        kps = (kps + BK * groups - 1) / (BK * groups) * (BK * groups);
        g.splits = splits = int((k + kps - 1) / kps);
        g.k_per_split = kps;
        g.partial = use.ptr();
        if (!g.partial) return CTAMD_EINVAL;
        if (size_t(tiles - whole_tiles) * size_t(splits) * size_t(BM) * size_t(BN) > kScratchFloats)
            return fail(CTAMD_ERANGE, "%s: the parts of %d split tiles do not fit the device scratch", name, tiles - whole_tiles);
    }
    // a tile outside [0, whole_tiles) writes its parts to g.partial: there is none unless the plan cut K
    if (splits == 1 && whole_tiles != tiles) return fail(CTAMD_EINVAL, "%s: plan leaves %d tiles without a part buffer", name, tiles - whole_tiles);
    const int blocks = whole_tiles + (tiles - whole_tiles) * splits;
    // b's column sums ride along when the product is cut along K on the 64 x 64 tile (the weight gradient
    // of a layer a few hundred wide at a large batch): stage 1 as extra blocks of the product's launch,
    // stage 2 as extra blocks of the launch that adds the parts - two launches fewer, the same bits
    if (sums && sums_done && splits > 1 && shape == 0 && groups == 1 && vec && !B_KC && bs0 == n &&
        colsum_narrow_plan(size_t(k), size_t(n), true, &g.sum) &&
        size_t(tiles - whole_tiles) * size_t(splits) * size_t(BM) * size_t(BN) + size_t(g.sum.chunks) * size_t(n) <= kScratchFloats) {
        g.sum_out = sums;
        g.sum_partials = g.partial + size_t(tiles - whole_tiles) * size_t(splits) * size_t(BM) * size_t(BN);
        g.product_blocks = blocks;
        *sums_done = true;
        account(4.0 * double(k) * double(n), double(k) * double(n), true);
        const int all = blocks + int(g.sum.chunks);
        int rc = blocks <= cus ? launch_with_sums<TinyEarlyTile>(g, A_KC, all, s) : launch_with_sums<TinyTile>(g, A_KC, all, s);
        if (rc) return rc;
        constexpr unsigned kFoldCols = kColsumThreads / kFoldLanes;
        const dim3 fold_grid(unsigned(tiles - whole_tiles) + (unsigned(n) + kFoldCols - 1) / kFoldCols, unsigned(BM * BN / kFoldSlice));
        hipLaunchKernelGGL((fold_parts<TinyTile::BM, TinyTile::BN>), fold_grid, dim3(kThreads), 0, s, g);
        return launched(name);
    }
    int rc = groups == 4 ? launch_layout<TinyK4Tile>(g, A_KC, B_KC, vec, blocks, s)
           : groups == 2 ? launch_gemm<Small16Tile, true, true>(g, vec, blocks, s)
           : (shape == 1 && blocks <= cus) ? launch_layout<Small8Tile>(g, A_KC, B_KC, vec, blocks, s)
           : (shape == 2 && A_KC && B_KC) ? launch_gemm<Big16Tile, true, true>(g, vec, blocks, s)
           : (shape == 2 && !A_KC && !B_KC) ? launch_gemm<Big16Tile, false, false>(g, vec, blocks, s)
           : (shape == 0 && blocks <= cus) ? launch_layout<TinyEarlyTile>(g, A_KC, B_KC, vec, blocks, s)
           : shape == 3 ? launch_layout<WideTile>(g, A_KC, B_KC, vec, blocks, s)
           : shape == 2 ? launch_layout<BigTile>(g, A_KC, B_KC, vec, blocks, s)
           : shape == 1 ? launch_layout<SmallTile>(g, A_KC, B_KC, vec, blocks, s)
                        : launch_layout<TinyTile>(g, A_KC, B_KC, vec, blocks, s);
    if (rc || splits == 1) return rc;
    const dim3 fold_grid(unsigned(tiles - whole_tiles), unsigned(BM * BN / kFoldSlice));
    if (shape == 3) hipLaunchKernelGGL((fold_parts<WideTile::BM, WideTile::BN>), fold_grid, dim3(kThreads), 0, s, g);
    else if (shape == 2) hipLaunchKernelGGL((fold_parts<BigTile::BM, BigTile::BN>), fold_grid, dim3(kThreads), 0, s, g);
    else if (shape == 1) hipLaunchKernelGGL((fold_parts<SmallTile::BM, SmallTile::BN>), fold_grid, dim3(kThreads), 0, s, g);
    else hipLaunchKernelGGL((fold_parts<TinyTile::BM, TinyTile::BN>), fold_grid, dim3(kThreads), 0, s, g);
    return launched(name);
}

}  // namespace

extern "C" int ctamd_matmul_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                                float* c, int64_t m, int64_t n, int64_t k, void* stream) {
    return matmul_impl(__func__, a, as0, as1, b, bs0, bs1, nullptr, 0, nullptr, c, m, n, k, stream);
}

extern "C" int ctamd_matmul_bias_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                                     const float* bias, int relu, float* c, int64_t m, int64_t n, int64_t k,
                                     void* stream) {
    return matmul_impl(__func__, a, as0, as1, b, bs0, bs1, bias, relu ? 1 : 0, nullptr, c, m, n, k, stream);
}

extern "C" int ctamd_matmul_colsum_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                                       float* c, float* sums, int64_t m, int64_t n, int64_t k, void* stream) {
    if (m < 0 || n < 0 || k < 0) return fail(CTAMD_EINVAL, "%s: negative extent", __func__);
    if (n > 0 && !sums) return fail(CTAMD_EINVAL, "%s: null sums", __func__);
    if ((n > 1 && bs1 != 1) || (k > 1 && bs0 != n))
        return fail(CTAMD_EINVAL, "%s: the column sums need b in contiguous rows (strides %lld, %lld)", __func__, (long long)bs0,
                    (long long)bs1);
    bool done = false;
    int rc = matmul_impl(__func__, a, as0, as1, b, bs0, bs1, nullptr, 0, nullptr, c, m, n, k, stream, sums, &done);
    if (rc || done || n == 0) return rc;
    return ctamd_colsum_f32(b, sums, size_t(k), size_t(n), stream);
}

extern "C" int ctamd_matmul_relu_mask_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                                          const float* y, float* c, int64_t m, int64_t n, int64_t k, void* stream) {
    if (m > 0 && n > 0 && !y) return fail(CTAMD_EINVAL, "%s: null activation", __func__);
    return matmul_impl(__func__, a, as0, as1, b, bs0, bs1, nullptr, 0, y, c, m, n, k, stream);
}
