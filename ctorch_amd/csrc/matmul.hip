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
#include "common.h"


namespace ctamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kXcds = 8;

constexpr int kMinWavesPerSimd = 2;   // register budget of both tile shapes: 256 VGPRs per lane


template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct Cfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int TM = WM / 32, TN = WN / 32;       // MFMA tiles per wave
    static constexpr int WAVES_N = BN / WN;
    static constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
    static_assert(THREADS == 256 || THREADS == 512, "4 or 8 waves per block");
    static_assert(BK % 8 == 0, "k tile is a multiple of the 8-wide chunk");
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
};

// Output epilogue of a product that is not split along K: bias add, then ReLU as `v > 0 ? v : +0`
// (NaN -> 0, -0 -> +0), each rounded as the separate Add and ReLU kernels round them, so that the
// fused product equals the three launches bit for bit.
__device__ __forceinline__ float epilogue(float v, const float* __restrict__ bias, int col, int relu) {
    if (bias) v = v + bias[col];
    if (relu) v = v > 0.0f ? v : 0.0f;
    return v;
}

template <class C, bool A_KC, bool B_KC, bool VEC>
__global__ __launch_bounds__(C::THREADS, kMinWavesPerSimd) void gemm_kernel(GemmArgs g) {
    constexpr int BM = C::BM, BN = C::BN, BK = C::BK, TM = C::TM, TN = C::TN;
    constexpr int A_STRIDE = A_KC ? C::KPAD : C::XPAD_M;
    constexpr int B_STRIDE = B_KC ? C::KPAD : C::XPAD_N;
    constexpr int A_FLOATS = tile_floats<C, A_KC, true>();
    constexpr int B_FLOATS = tile_floats<C, B_KC, false>();
    __shared__ __attribute__((aligned(16))) float s_a[2][A_FLOATS];
    __shared__ __attribute__((aligned(16))) float s_b[2][B_FLOATS];

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

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
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
    // interior: the whole BM x BN tile and every k tile lie inside the operands and rows are
    // 16-byte aligned - true for all blocks of a 4096^3 product, false only on ragged edges
    const bool interior = VEC && m0 + BM <= g.m && n0 + BN <= g.n && (k_end - k_begin) % BK == 0 &&
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
    constexpr int NCH = BK / 8;
    static_assert(NCH == 2, "the pipeline below alternates two fragment buffers over two chunks");
    float fa[2][TM][4], fb[2][TN][4];
    auto fetch_chunk = [&](int buf, int ch, int which) {
        const float* __restrict__ la = s_a[buf];
        const float* __restrict__ lb = s_b[buf];
        const int kb = ch * 8 + half * 4;
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
        for (int t = 0; t + 1 < ktiles; ++t) {
            const int cur = t & 1;
            __builtin_amdgcn_sched_barrier(0);
            lds_wait();
            fetch_chunk(cur, 1, 1);
            mfmas(0);
            sa.store(s_a[cur ^ 1], A_STRIDE);
            sb.store(s_b[cur ^ 1], B_STRIDE);
#pragma unroll
            for (int q = 0; q < kReadSlots; ++q) {
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 0);
                __builtin_amdgcn_sched_group_barrier(kMaskDsRead, 1, 0);
            }
            if (kMfmaPerChunk - kReadSlots - kStores > 0)
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, kMfmaPerChunk - kReadSlots - kStores, 0);
#pragma unroll
            for (int q = 0; q < kStores; ++q) {
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 0);
                __builtin_amdgcn_sched_group_barrier(kMaskDsWrite, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            fetch_chunk(cur ^ 1, 0, 0);
            const bool more = t + 3 < ktiles;
            sa.load_fast(more ? a_step : 0);
            sb.load_fast(more ? b_step : 0);
            mfmas(1);
#pragma unroll
            for (int q = 0; q < kReadSlots; ++q) {
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 1);
                __builtin_amdgcn_sched_group_barrier(kMaskDsRead, 1, 1);
            }
#pragma unroll
            for (int q = 0; q < kStores; ++q) {
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, 1, 1);
                __builtin_amdgcn_sched_group_barrier(kMaskVmemRead, 1, 1);
            }
            if (kMfmaPerChunk - kReadSlots - kStores > 0)
                __builtin_amdgcn_sched_group_barrier(kMaskMfma, kMfmaPerChunk - kReadSlots - kStores, 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
        auto stage_tile = [&](int t) {
            sa.template load<VEC>(g.a, g.lda, m0, k_begin + t * BK, g.m, k_end);
            sb.template load<VEC>(g.b, g.ldb, n0, k_begin + t * BK, g.n, k_end);
        };
        stage_tile(0);
        sa.store(s_a[0], A_STRIDE);
        sb.store(s_b[0], B_STRIDE);
        __syncthreads();
        if (ktiles > 1) stage_tile(1);
        fetch_chunk(0, 0, 0);
        for (int t = 0; t + 1 < ktiles; ++t) {
            const int cur = t & 1;
            lds_wait();
            fetch_chunk(cur, 1, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfmas(0);
            __builtin_amdgcn_sched_barrier(0);
            sa.store(s_a[cur ^ 1], A_STRIDE);
            sb.store(s_b[cur ^ 1], B_STRIDE);
            __syncthreads();
            fetch_chunk(cur ^ 1, 0, 0);
            if (t + 2 < ktiles) stage_tile(t + 2);
            __builtin_amdgcn_sched_barrier(0);
            mfmas(1);
            __builtin_amdgcn_sched_barrier(0);
        }
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
                    if (row < g.m && col < g.n) g.c[int64_t(row) * g.ldc + col] = epilogue(acc[i][j][r], g.bias, col, g.relu);
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

// Adds the parts of the split tiles in their order and writes C (bias and ReLU of the fused
// product included): blockIdx.x is the split tile, blockIdx.y one of its slices of kFoldSlice elements.
constexpr int kFoldSlice = kThreads * 4;       // one 128-bit word per thread: a tile cut in many parts has few tiles, and the grid is tiles x slices
template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void fold_parts(GemmArgs g) {
    static_assert(BM * BN % kFoldSlice == 0, "a tile is a whole number of slices");
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
            if (gcol + e < g.n) t[e] = epilogue(t[e], g.bias, gcol + e, g.relu);
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

template <class Tile, bool A_KC, bool B_KC>
int launch_gemm(GemmArgs g, bool vec, int blocks, hipStream_t s) {
    if (vec) hipLaunchKernelGGL((gemm_kernel<Tile, A_KC, B_KC, true>), dim3(unsigned(blocks)), dim3(Tile::THREADS), 0, s, g);
    else hipLaunchKernelGGL((gemm_kernel<Tile, A_KC, B_KC, false>), dim3(unsigned(blocks)), dim3(Tile::THREADS), 0, s, g);
    return launched("ctamd_matmul_f32");
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
int matmul_impl(const char* name, const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                const float* bias, int relu, float* c, int64_t m, int64_t n, int64_t k, void* stream) {
    if (m < 0 || n < 0 || k < 0) return fail(CTAMD_EINVAL, "%s: negative extent", name);
    if (m == 0 || n == 0) return CTAMD_OK;
    if (!c) return fail(CTAMD_EINVAL, "%s: null output", name);
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff || m * n > (int64_t(1) << 40))
        return fail(CTAMD_ERANGE, "%s: extent too large", name);
    if (k == 0) {                                   // an empty sum: 0, then the epilogue
        int rc = ctamd_fill_f32(c, 0.0f, size_t(m) * size_t(n), stream);
        if (!rc && bias) rc = ctamd_add_rowbcast_f32(c, bias, c, size_t(m), size_t(n), stream);
        if (!rc && relu) rc = ctamd_relu_f32(c, c, size_t(m) * size_t(n), stream);
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
        return launched(name);
    }
    const bool A_KC = a_kc, B_KC = !b_xc;
    const int cus = compute_units() > 0 ? compute_units() : 256;
    constexpr int BK = 16;
    static_assert(BigTile::BK == BK && WideTile::BK == BK && SmallTile::BK == BK && TinyTile::BK == BK, "all tile shapes step K alike");
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
    struct Shape { int bm, bn, together; double per_flop, alone; };
    static const Shape shapes[4] = {{TinyTile::BM, TinyTile::BN, 4, 1.30, 1.70}, {SmallTile::BM, SmallTile::BN, 2, 1.07, 1.34},
                                    {BigTile::BM, BigTile::BN, 1, 1.00, 1.00}, {WideTile::BM, WideTile::BN, 2, 1.04, 1.32}};
    const double t_elem = 2.0 * double(k) / (157.3e12 * 0.92 / cus);
    int shape = 0, splits = 1, whole_tiles = 0;
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
        for (int parts : {1, most / 2, most}) {
            if (parts < 1 || (parts == 1 && most > 1 && left == 0)) continue;
            double cost = double(rounds) * q.together * q.per_flop * area * t_elem;
            if (left > 0) {
                const int64_t c = (left * parts + cus - 1) / cus;
                const double busy = q.together == 1 ? q.alone
                                                    : q.alone + double(c - 1) * (q.together * q.per_flop - q.alone) / (q.together - 1);
                cost += busy * area * t_elem / parts + (rounds == 0 ? 3e-6 : 1e-6);
                if (parts > 1) cost += 6e-6 + double(left) * parts * area * 8.0 / 4e12;
            }
            if (best < 0.0 || cost < best) {
                best = cost; shape = sh; splits = parts; whole_tiles = int(parts > 1 ? tiles - left : tiles);
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
    g.bias = bias; g.relu = relu;
    g.c_vec = (aligned16(c) && n % 4 == 0) ? 1 : 0;
    const bool vec = aligned16(a) && aligned16(b) && (g.lda % 4 == 0) && (g.ldb % 4 == 0);
    const int tiles = g.tiles_m * g.tiles_n;
    g.whole_tiles = whole_tiles;
    g.splits = splits;
    g.partial = nullptr;
    g.k_per_split = int(k);
    if (splits > 1) {
        int kps = int((k + splits - 1) / splits);
        kps = (kps + BK - 1) / BK * BK;
        g.splits = splits = int((k + kps - 1) / kps);
        g.k_per_split = kps;
        g.partial = scratch(stream);
        if (!g.partial) return CTAMD_EINVAL;
        if (size_t(tiles - whole_tiles) * size_t(splits) * size_t(BM) * size_t(BN) > kScratchFloats)
            return fail(CTAMD_ERANGE, "%s: the parts of %d split tiles do not fit the device scratch", name, tiles - whole_tiles);
    }
    const int blocks = whole_tiles + (tiles - whole_tiles) * splits;
    int rc = shape == 3 ? launch_layout<WideTile>(g, A_KC, B_KC, vec, blocks, s)
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
    return matmul_impl(__func__, a, as0, as1, b, bs0, bs1, nullptr, 0, c, m, n, k, stream);
}

extern "C" int ctamd_matmul_bias_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                                     const float* bias, int relu, float* c, int64_t m, int64_t n, int64_t k,
                                     void* stream) {
    return matmul_impl(__func__, a, as0, as1, b, bs0, bs1, bias, relu ? 1 : 0, c, m, n, k, stream);
}
