// The classifier head of a small network in one pass over the hidden activations: for every row of
// h [B x H], with at most 16 classes and H <= 256,
//     z = h . W + b                          (mnist/mnist.cpp:41: the last layer)
//     loss -= log(max(softmax(z)[label], 1e-10))   (CrossEntropy_BASIC_kernel.cpp:88-120, summed over rows)
//     dz = softmax(z) - onehot(label)        (src/AutoDiff.cpp:1517-1601 for an upstream gradient of 1)
//     dh = (dz . W^T) [* (h > 0)]            (src/AutoDiff.cpp:1684-1704, and the ReLU branch :1320-1371
//                                             of the layer that produced h)
//     gW += h^T . dz,  gb += dz              (src/AutoDiff.cpp:1766-1810; the bias as a column sum)
// which the operator-by-operator step computes in five launches whose work is a few microseconds each.
// A product with ten output columns cannot use the matrix cores (a 32 x 32 tile would be two thirds
// idle); everything here is fp32 fused multiply-adds on the vector units, h read once, dh written once.
//
// A wave takes four rows at a time (two when there are more than 13 classes).  Lane l holds h[row][4l .. 4l+3] and the four rows of W those k
// meet (W stays in registers for all rows); the 4 x N partial logits go round the wave with the
// halving exchange of the narrow products (lane r * N + c ends up with z[r][c]); the N lanes of a row
// form its softmax by lane reads; dz comes back to every lane through scalar lane reads and meets h
// and W in registers once more for dh and for the wave's share of gW.  The shares of the block's eight
// waves are added in wave order through LDS; every block leaves gW, gb, its loss (a double) and a
// bad-label flag in the device scratch, and a second launch adds the blocks in block order
// (deterministic; 16 lanes per element).
#include "common.h"
#include "devmath.h"

namespace ctamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

// waves per block: eight (two per SIMD, whose exchanges and lane reads hide each other's latency) while
// the kernel fits 256 registers per lane at that occupancy, four for the widest heads
constexpr int head_waves(int n) { return n <= 13 ? 8 : 4; }
// rows a wave works on at a time (their partial logits share one exchange): four, two for the widest heads
constexpr int head_rows(int n) { return n <= 13 ? 4 : 2; }
constexpr int kHeadMaxBlocks = 256;       // partial results kept per launch
constexpr int kHeadMaxH = 256;

struct HeadArgs {
    const float* h;          // [B, H] row-major
    const float* w;          // [H, N] row-major
    const float* bias;       // [N]
    const float* labels;     // [B] class indices as floats
    float* z;                // [B, N] logits (may be null)
    float* dz;               // [B, N]
    float* dh;               // [B, H] (may be null)
    float* part;             // scratch: per block [H * N] + [N] floats, then per block {double loss, double bad}
    int B, H;
    int turns;               // groups of rows per wave
    int mask;                // dh is multiplied by (h > 0 ? 1 : 0)
    int fast;                // single-precision exponential and e * (1 / s), as the row kernels' default mode
};

constexpr int pow2_at_least_(int v) { return v <= 1 ? 1 : 2 * pow2_at_least_((v + 1) / 2); }

template <int CNT, int OFF, int P>
__device__ __forceinline__ void wave_sums_step_(float (&v)[P], int lane) {
    if constexpr (CNT > 1) {
        const bool upper = (lane & OFF) != 0;
#pragma unroll
        for (int j = 0; j < CNT / 2; ++j) {
            const float send = upper ? v[j] : v[j + CNT / 2];
            const float keep = upper ? v[j + CNT / 2] : v[j];
            v[j] = keep + __shfl_xor(send, OFF, 64);
        }
        wave_sums_step_<CNT / 2, OFF / 2, P>(v, lane);
    } else if constexpr (OFF >= 1) {
        v[0] = v[0] + __shfl_xor(v[0], OFF, 64);
        wave_sums_step_<1, OFF / 2, P>(v, lane);
    }
}

__host__ __device__ inline size_t head_part_floats(int H, int N) { return size_t(H) * N + N; }

template <int N>
__global__ __launch_bounds__(head_waves(N) * 64) void head_kernel(HeadArgs a) {
    constexpr int kHeadWaves = head_waves(N);
    constexpr int kHeadThreads = kHeadWaves * 64;
    constexpr int R = head_rows(N);
    constexpr int P = pow2_at_least_(R * N);
    constexpr int kLanesPerValue = 64 / P;
    __shared__ __attribute__((aligned(16))) float s_wt[N][kHeadMaxH];     // W transposed, zeros behind H
    __shared__ uint64_t s_exp2[32];
    __shared__ float s_gw[64][4 * N + 1];                                 // the waves' shares of gW, added in wave order
    __shared__ float s_gb[kHeadWaves][N];
    __shared__ double s_loss[kHeadWaves];
    __shared__ int s_bad[kHeadWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int H = a.H;
    const int kk = 4 * lane;
    const bool k_ok = kk < H;                                             // H is a multiple of four

    auto load_rows = [&](int row0, v4f (&hv)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (k_ok && row0 + r < a.B) v = *reinterpret_cast<const v4f*>(a.h + size_t(row0 + r) * H + kk);
            hv[r] = v;
        }
    };
    const int first = (blockIdx.x * kHeadWaves * a.turns + wave) * R;
    const int stride = kHeadWaves * R;
    v4f hv[R];
    load_rows(first, hv);                                                 // on its way while W is staged
    for (int e = threadIdx.x; e < kHeadMaxH * N; e += kHeadThreads) {
        const int k = e / N, c = e % N;
        s_wt[c][k] = k < H ? a.w[size_t(k) * N + c] : 0.0f;
    }
    if (threadIdx.x < 32) s_exp2[threadIdx.x] = cta_exp2_tab[threadIdx.x];
    __syncthreads();
    v4f wv[N];
#pragma unroll
    for (int c = 0; c < N; ++c) wv[c] = *reinterpret_cast<const v4f*>(&s_wt[c][kk]);

    // which value of the exchange this lane ends up with: row v / N of the group, class v % N
    const int v_mine = lane / kLanesPerValue;
    const bool holder = (lane % kLanesPerValue == 0) && v_mine < R * N;
    const int r_mine = holder ? v_mine / N : 0, c_mine = holder ? v_mine % N : 0;
    const float bias_mine = holder ? a.bias[c_mine] : 0.0f;

    float gw[4][N];                     // this wave's share of gW[4l + e][c]
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int c = 0; c < N; ++c) gw[e][c] = 0.0f;
    float gb_mine = 0.0f;               // sum of dz over this lane's (row of the group, class), all turns
    double loss_mine = 0.0;
    bool bad = false;

    for (int t = 0; t < a.turns; ++t) {
        const int row0 = first + t * stride;
        if (row0 >= a.B) break;                                           // wave-uniform
        v4f next[R];
        const bool more = t + 1 < a.turns && row0 + stride < a.B;
        if (more) load_rows(row0 + stride, next);
        float acc[P];
#pragma unroll
        for (int v = 0; v < P; ++v) acc[v] = 0.0f;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < N; ++c)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[r * N + c] = __fmaf_rn(hv[r][e], wv[c][e], acc[r * N + c]);
        wave_sums_step_<P, 32, P>(acc, lane);
        // lane (r * N + c) * kLanesPerValue holds the product's element; the bias joins as a separate add
        const float z_mine = acc[0] + bias_mine;
        const int row_mine = row0 + r_mine;
        const bool live = holder && row_mine < a.B;
        // the row's softmax among its N lanes
        float zr[N];
#pragma unroll
        for (int c = 0; c < N; ++c) zr[c] = __shfl(z_mine, (r_mine * N + c) * kLanesPerValue, 64);
        float m = zr[0];
#pragma unroll
        for (int c = 1; c < N; ++c) m = zr[c] > m ? zr[c] : m;
        const float e_mine = a.fast ? cta_exp_hw_nonpos(z_mine - m) : cta_expf_nonpos(z_mine - m, s_exp2);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < N; ++c) s = s + __shfl(e_mine, (r_mine * N + c) * kLanesPerValue, 64);
        const float sm = a.fast ? e_mine * (1.0f / s) : cta_div_rcp(e_mine, 1.0 / double(s));
        const int label = live ? class_index(a.labels[row_mine]) : 0;
        const bool label_ok = label >= 0 && label < N;
        const bool is_class = live && label_ok && label == c_mine;
        const float dz_mine = live ? 0.0f + (sm - (is_class ? 1.0f : 0.0f)) : 0.0f;
        if (live && !label_ok && c_mine == 0) {
            bad = true;
            loss_mine += double(__builtin_nanf(""));
        }
        if (is_class) {
            float p = e_mine / s;
            p = (p < 1e-10f) ? 1e-10f : p;
            loss_mine -= double(float(log(double(p))));
        }
        if (live) {
            if (a.z) a.z[size_t(row_mine) * N + c_mine] = z_mine;
            a.dz[size_t(row_mine) * N + c_mine] = dz_mine;
        }
        gb_mine += dz_mine;
        // dz of the rows to every lane (scalar lane reads), then dh and the share of gW
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float d[N];
#pragma unroll
            for (int c = 0; c < N; ++c) d[c] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(dz_mine), (r * N + c) * kLanesPerValue));
            v4f out = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float sum = 0.0f;
#pragma unroll
                for (int c = 0; c < N; ++c) {
                    sum = __fmaf_rn(d[c], wv[c][e], sum);
                    gw[e][c] = __fmaf_rn(hv[r][e], d[c], gw[e][c]);
                }
                out[e] = a.mask ? sum * (hv[r][e] > 0.0f ? 1.0f : 0.0f) : sum;
            }
            if (a.dh && k_ok && row0 + r < a.B) *reinterpret_cast<v4f*>(a.dh + size_t(row0 + r) * H + kk) = out;
        }
        if (more) {
#pragma unroll
            for (int r = 0; r < R; ++r) hv[r] = next[r];
        }
    }

    // the block's shares: waves added in wave order (wave 0 writes, the others add in turn)
    for (int w = 0; w < kHeadWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int c = 0; c < N; ++c) {
                    float& at = s_gw[lane][e * N + c];
                    at = (w == 0) ? gw[e][c] : at + gw[e][c];
                }
        }
        __syncthreads();
    }
    // a lane's gb share belongs to class c_mine; the R rows of the group are R lanes apart in steps of N values
    float gb_c = 0.0f;
    {
        // lanes holding (r, c) for r = 0 .. R-1, added in order of r by the lane with r == 0
        float parts[R];
#pragma unroll
        for (int r = 0; r < R; ++r) parts[r] = __shfl(gb_mine, ((r * N + c_mine) * kLanesPerValue) & 63, 64);
#pragma unroll
        for (int r = 0; r < R; ++r) gb_c = gb_c + parts[r];
    }
    if (holder && r_mine == 0) s_gb[wave][c_mine] = gb_c;
    // the wave's loss and flag
    for (int off = 32; off > 0; off >>= 1) loss_mine += __shfl_xor(loss_mine, off, 64);
    const bool any_bad = __any(bad);
    if (lane == 0) {
        s_loss[wave] = loss_mine;
        s_bad[wave] = any_bad ? 1 : 0;
    }
    __syncthreads();
    float* __restrict__ mine = a.part + size_t(blockIdx.x) * head_part_floats(H, N);
    for (int i = threadIdx.x; i < H * N; i += kHeadThreads) {
        const int k = i / N, c = i % N;
        mine[i] = s_gw[k / 4][(k % 4) * N + c];
    }
    if (threadIdx.x < N) {
        float t = s_gb[0][threadIdx.x];
#pragma unroll
        for (int w = 1; w < kHeadWaves; ++w) t = t + s_gb[w][threadIdx.x];
        mine[size_t(H) * N + threadIdx.x] = t;
    }
    if (threadIdx.x == 0) {
        double* tail = reinterpret_cast<double*>(a.part + size_t(gridDim.x) * head_part_floats(H, N) + (head_part_floats(H, N) * gridDim.x) % 2);
        double l = 0.0;
        int b = 0;
        for (int w = 0; w < kHeadWaves; ++w) {
            l += s_loss[w];
            b |= s_bad[w];
        }
        tail[2 * blockIdx.x] = l;
        tail[2 * blockIdx.x + 1] = b ? 1.0 : 0.0;
    }
}

// Adds the blocks' shares in block order.  A block of 256 threads owns 16 neighbouring elements of
// [gW | gb]: thread (slice s, element e) adds blocks s, s + 16, s + 32, ... in that order, sixteen
// loads in flight at a time, and the sixteen slices are added in slice order through LDS.  The first
// thread of the launch adds the blocks' losses and flags.
constexpr int kFoldThreads = 256;
__global__ __launch_bounds__(kFoldThreads) void head_fold_kernel(const float* __restrict__ part, int blocks, int per_block, int gw_elems,
                                                                  float* __restrict__ gw, float* __restrict__ gb, float* __restrict__ loss,
                                                                  int32_t* __restrict__ status) {
    __shared__ float s_t[16][17];
    const int e = threadIdx.x % 16, s = threadIdx.x / 16;
    const int elem = blockIdx.x * 16 + e;
    float t = 0.0f;
    if (elem < per_block) {
        for (int base = 0; base < blocks; base += 256) {
            float v[16];
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int b = base + s + 16 * q;
                v[q] = b < blocks ? part[size_t(b) * per_block + elem] : 0.0f;
            }
#pragma unroll
            for (int q = 0; q < 16; ++q) t = t + v[q];
        }
    }
    s_t[s][e] = t;
    __syncthreads();
    if (s == 0 && elem < per_block) {
        float sum = s_t[0][e];
#pragma unroll
        for (int q = 1; q < 16; ++q) sum = sum + s_t[q][e];
        if (elem < gw_elems) gw[elem] = sum;
        else gb[elem - gw_elems] = sum;
    }
    // the blocks' losses and flags: the last wave of the first block, lane l adds blocks l, l + 64, ...
    // in order (at most kHeadMaxBlocks / 64 loads each, all in flight), then the lanes in a fixed tree
    if (blockIdx.x == 0 && threadIdx.x >= kFoldThreads - 64) {
        const int lane = threadIdx.x & 63;
        const double* tail = reinterpret_cast<const double*>(part + size_t(blocks) * per_block + (size_t(per_block) * blocks) % 2);
        double v[kHeadMaxBlocks / 64], f[kHeadMaxBlocks / 64];
#pragma unroll
        for (int q = 0; q < kHeadMaxBlocks / 64; ++q) {
            const int b = lane + 64 * q;
            v[q] = b < blocks ? tail[2 * b] : 0.0;
            f[q] = b < blocks ? tail[2 * b + 1] : 0.0;
        }
        double l = 0.0, bad = 0.0;
#pragma unroll
        for (int q = 0; q < kHeadMaxBlocks / 64; ++q) {
            l += v[q];
            bad += f[q];
        }
        for (int off = 32; off > 0; off >>= 1) {
            l += __shfl_xor(l, off, 64);
            bad += __shfl_xor(bad, off, 64);
        }
        if (lane == 0) {
            loss[0] = float(l);
            if (status) status[0] = bad != 0.0 ? 1 : 0;
        }
    }
}

template <int N>
int launch_head(const HeadArgs& a, int blocks, hipStream_t s) {
    hipLaunchKernelGGL(head_kernel<N>, dim3(unsigned(blocks)), dim3(head_waves(N) * 64), 0, s, a);
    return launched("ctamd_linear_ce_head_f32");
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" int ctamd_linear_ce_head_fits(size_t hidden, size_t classes) {
    return (classes >= 2 && classes <= 16 && hidden >= 4 && hidden <= size_t(kHeadMaxH) && hidden % 4 == 0) ? 1 : 0;
}

extern "C" int ctamd_linear_ce_head_f32(const float* h, const float* w, const float* bias, const float* labels, float* loss, int32_t* status,
                                        float* z, float* dz, float* dh, int mask_by_h, float* gw, float* gb, size_t batch, size_t hidden,
                                        size_t classes, void* stream) {
    if (!ctamd_linear_ce_head_fits(hidden, classes))
        return fail(CTAMD_ERANGE, "%s: needs 2 to 16 classes and a hidden width of 4 to %d that is a multiple of four", __func__, kHeadMaxH);
    if (batch == 0 || batch > 0x3fffffffu) return fail(CTAMD_ERANGE, "%s: batch out of range", __func__);
    if (!h || !w || !bias || !labels || !loss || !dz || !gw || !gb) return fail(CTAMD_EINVAL, "%s: null pointer", __func__);
    if (!aligned16(h) || (dh && !aligned16(dh))) return fail(CTAMD_EINVAL, "%s: h and dh must be 16-byte aligned", __func__);
    ScratchUse use(stream);
    float* part = use.ptr();
    if (!part) return CTAMD_EINVAL;
    const int B = int(batch), H = int(hidden), N = int(classes);
    const int rows_at_a_time = head_rows(N);
    const int groups = (B + rows_at_a_time - 1) / rows_at_a_time;       // groups of rows a wave takes together
    const int waves = head_waves(N);
    const int cus = compute_units() > 0 ? compute_units() : 256;
    int blocks = (groups + waves - 1) / waves;
    const int cap = cus < kHeadMaxBlocks ? cus : kHeadMaxBlocks;
    if (blocks > cap) blocks = cap;
    const int turns = (groups + blocks * waves - 1) / (blocks * waves);
    blocks = (groups + turns * waves - 1) / (turns * waves);
    if ((head_part_floats(H, N) + 4) * size_t(blocks) + 2 > kScratchFloats) return fail(CTAMD_ERANGE, "%s: does not fit the device scratch", __func__);
    HeadArgs a;
    a.h = h; a.w = w; a.bias = bias; a.labels = labels; a.z = z; a.dz = dz; a.dh = dh; a.part = part;
    a.B = B; a.H = H; a.turns = turns; a.mask = mask_by_h ? 1 : 0; a.fast = fast_math() ? 1 : 0;
    hipStream_t s = as_stream(stream);
    int rc = CTAMD_EINVAL;
    switch (N) {
        case 2: rc = launch_head<2>(a, blocks, s); break;
        case 3: rc = launch_head<3>(a, blocks, s); break;
        case 4: rc = launch_head<4>(a, blocks, s); break;
        case 5: rc = launch_head<5>(a, blocks, s); break;
        case 6: rc = launch_head<6>(a, blocks, s); break;
        case 7: rc = launch_head<7>(a, blocks, s); break;
        case 8: rc = launch_head<8>(a, blocks, s); break;
        case 9: rc = launch_head<9>(a, blocks, s); break;
        case 10: rc = launch_head<10>(a, blocks, s); break;
        case 11: rc = launch_head<11>(a, blocks, s); break;
        case 12: rc = launch_head<12>(a, blocks, s); break;
        case 13: rc = launch_head<13>(a, blocks, s); break;
        case 14: rc = launch_head<14>(a, blocks, s); break;
        case 15: rc = launch_head<15>(a, blocks, s); break;
        case 16: rc = launch_head<16>(a, blocks, s); break;
        default: break;
    }
    if (rc) return rc;
    const int per_block = int(head_part_floats(H, N));
    hipLaunchKernelGGL(head_fold_kernel, dim3(unsigned((per_block + 15) / 16)), dim3(kFoldThreads), 0, s, part, blocks, per_block, H * N, gw, gb,
                       loss, status);
    // what the five launches this replaces must move and compute: h read, dh written, the small
    // operands; three products of 2 B H N flop
    account(4.0 * (double(B) * H * (dh ? 2.0 : 1.0) + 2.0 * double(H) * N + 3.0 * double(B) * N), 6.0 * double(B) * double(H) * double(N));
    return launched(__func__);
}
