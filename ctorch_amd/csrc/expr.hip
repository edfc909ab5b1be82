// Fused elementwise expressions: a straight-line program of the per-element operators (the same
// functors the one-operator kernels use) evaluated in ONE pass over memory - every input is read
// once, every output written once, intermediates never leave the chip.  The front-end compiles
// both an expression's forward values and its tape gradients into such programs, so a chain like
// Y = sigmoid(X / r) - tanh(X) * sin(X) + cos(-X) is one launch forward and one launch backward
// instead of nine and about fifteen, with the bits of the operator-by-operator evaluation.
//
// The kernel is an interpreter: the program sits in the kernel arguments (uniform, read through
// the scalar unit), so every instruction is a scalar branch to one functor's code, applied to the
// four elements each lane owns.  Values live in LDS "slots": slot s of element e of lane t at
// slots[(s * 4 + e) * 256 + t] - consecutive lanes on consecutive banks, no conflicts.  An
// instruction costs two LDS reads and one write per element next to its arithmetic; for the
// transcendental operators that is noise, for a chain of cheap operators the kernel stays bound by
// the memory stream.  (Registers cannot hold the slots: the slot number is data.)
#include "common.h"
#include "devmath.h"
#include "functors.h"

#include <cfloat>

namespace ctamd {
namespace {

constexpr int kExprThreads = 256;
constexpr int kPerLane = 4;                   // elements per lane and pass
constexpr int kMaxInsns = CTAMD_EXPR_MAX_INSNS;
constexpr int kMaxSlots = CTAMD_EXPR_MAX_SLOTS;
constexpr int kMaxPorts = CTAMD_EXPR_MAX_PORTS;
constexpr int kMaxDevices = 64;

struct DevInsn {
    uint8_t op, dst, a, b;
    float imm;
    double rcp;                               // DIVS: 1 / double(imm)
};

struct ExprArgs {
    const float* in[kMaxPorts];
    float* out[kMaxPorts];
    int32_t* status;
    size_t total;                             // elements of a full-shape value
    unsigned cols;                            // row length (row-vector loads)
    int n_insn;
    int vec;                                  // 1: 128-bit accesses (all pointers aligned, total % 4 == 0, cols % 4 == 0)
    int has_row;                              // the program loads a row vector
    DevInsn prog[kMaxInsns];
};

// One operator on the four elements of a lane; a, b are the operand values.  The operator is chosen
// once (a scalar branch) and its four evaluations are independent instruction streams that the
// compiler interleaves: the long dependent chains of the transcendental functors (fp64 inside
// sinf / cosf) hide each other's latencies.
template <class F>
__device__ __forceinline__ void each(float (&o)[kPerLane], F f) {
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) o[e] = f(e);
}
__device__ __forceinline__ void apply(const DevInsn& q, const float (&a)[kPerLane], const float (&b)[kPerLane],
                                      float (&o)[kPerLane], const Tables& t) {
    switch (q.op) {
        case CTAMD_EX_ADD: each(o, [&](int e) { return a[e] + b[e]; }); break;
        case CTAMD_EX_SUB: each(o, [&](int e) { return a[e] - b[e]; }); break;
        case CTAMD_EX_MUL: each(o, [&](int e) { return a[e] * b[e]; }); break;
        case CTAMD_EX_DIV: each(o, [&](int e) { return a[e] / b[e]; }); break;
        case CTAMD_EX_NEG: each(o, [&](int e) { return -a[e]; }); break;
        case CTAMD_EX_RELU: each(o, [&](int e) { return (0.0f < a[e]) ? a[e] : 0.0f; }); break;
        case CTAMD_EX_SIGMOID: each(o, [&](int e) { return sigmoid_ref(a[e], t); }); break;
        case CTAMD_EX_TANH: each(o, [&](int e) { return tanh_ref(a[e], t); }); break;
        case CTAMD_EX_SIN:
        case CTAMD_EX_COS: {
            const int want_cos = (q.op == CTAMD_EX_COS);
            bool rare = false;
#pragma unroll
            for (int e = 0; e < kPerLane; ++e) {
                o[e] = cta_sincosf_fast(a[e], want_cos);
                rare = rare || cta_sincos_is_rare(a[e]);
            }
            if (__builtin_expect(rare, 0)) {
                for (int e = 0; e < kPerLane; ++e)
                    if (cta_sincos_is_rare(a[e])) o[e] = cta_sincosf(a[e], want_cos, t.inv_pio4);
            }
            break;
        }
        case CTAMD_EX_ADDS: each(o, [&](int e) { return a[e] + q.imm; }); break;
        case CTAMD_EX_MULS: each(o, [&](int e) { return a[e] * q.imm; }); break;
        case CTAMD_EX_DIVS: each(o, [&](int e) { return cta_div_rcp(a[e], q.rcp); }); break;
        case CTAMD_EX_RSUBS: each(o, [&](int e) { return q.imm - a[e]; }); break;
        case CTAMD_EX_RELUMUL: each(o, [&](int e) { return b[e] * ((a[e] > 0.0f) ? 1.0f : 0.0f); }); break;
        default: each(o, [&](int e) { return a[e]; }); break;
    }
}

__global__ __launch_bounds__(kExprThreads) void expr_kernel(ExprArgs g) {
    extern __shared__ float slots[];          // [slots used][kPerLane][kExprThreads]
    __shared__ uint64_t s_exp2[32];
    __shared__ uint32_t s_pio4[24];
    stage_tables(s_exp2, s_pio4);
    const Tables tabs{s_exp2, s_pio4};
    const unsigned tid = threadIdx.x;
    const size_t per_pass = size_t(kExprThreads) * kPerLane;
    const size_t passes = (g.total + per_pass - 1) / per_pass;
    for (size_t pass = blockIdx.x; pass < passes; pass += gridDim.x) {
        // element e of this lane: vec - four consecutive elements (one 128-bit access);
        // else - elements 256 apart (coalesced 32-bit accesses)
        const size_t first = pass * per_pass + (g.vec ? size_t(tid) * kPerLane : size_t(tid));
        const size_t step = g.vec ? 1 : kExprThreads;
        const unsigned col_first = g.has_row ? unsigned(first % g.cols) : 0u;
        for (int pc = 0; pc < g.n_insn; ++pc) {
            const DevInsn q = g.prog[pc];
            float* __restrict__ d = slots + size_t(q.dst) * (kPerLane * kExprThreads) + tid;
            const float* __restrict__ pa = slots + size_t(q.a) * (kPerLane * kExprThreads) + tid;
            const float* __restrict__ pb = slots + size_t(q.b) * (kPerLane * kExprThreads) + tid;
            if (q.op == CTAMD_EX_LOAD_FULL) {
                const float* __restrict__ src = g.in[q.a];
                if (g.vec) {
                    if (first < g.total) {
                        v4f v = *reinterpret_cast<const v4f*>(src + first);
#pragma unroll
                        for (int e = 0; e < kPerLane; ++e) d[e * kExprThreads] = v[e];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < kPerLane; ++e) {
                        size_t i = first + size_t(e) * step;
                        if (i < g.total) d[e * kExprThreads] = src[i];
                    }
                }
            } else if (q.op == CTAMD_EX_LOAD_ROW) {
                const float* __restrict__ src = g.in[q.a];
                if (g.vec) {
                    if (first < g.total) {
                        v4f v = *reinterpret_cast<const v4f*>(src + col_first);
#pragma unroll
                        for (int e = 0; e < kPerLane; ++e) d[e * kExprThreads] = v[e];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < kPerLane; ++e) {
                        size_t i = first + size_t(e) * step;
                        if (i < g.total) d[e * kExprThreads] = src[(col_first + unsigned(e) * (kExprThreads % g.cols)) % g.cols];
                    }
                }
            } else if (q.op == CTAMD_EX_STORE || q.op == CTAMD_EX_STORE_ZP) {
                float* __restrict__ dst = g.out[q.dst];
                const bool zp = (q.op == CTAMD_EX_STORE_ZP);
                if (g.vec) {
                    if (first < g.total) {
                        v4f v;
#pragma unroll
                        for (int e = 0; e < kPerLane; ++e) {
                            float x = pa[e * kExprThreads];
                            v[e] = zp ? 0.0f + x : x;
                        }
                        *reinterpret_cast<v4f*>(dst + first) = v;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < kPerLane; ++e) {
                        size_t i = first + size_t(e) * step;
                        if (i < g.total) {
                            float x = pa[e * kExprThreads];
                            dst[i] = zp ? 0.0f + x : x;
                        }
                    }
                }
            } else if (q.op == CTAMD_EX_DIVCHK) {
                // the tape refuses to differentiate a division whose divisor has an element with
                // |b| < FLT_EPSILON (the reference: src/AutoDiff.cpp:1267-1284); reported through status
                bool bad = false;
                for (int e = 0; e < kPerLane; ++e) {
                    size_t i = first + size_t(e) * step;
                    if (i < g.total) bad = bad || (fabsf(pa[e * kExprThreads]) < FLT_EPSILON);
                }
                if (bad) atomicOr(g.status, 1);
            } else {
                // lanes past the end compute on whatever their slots hold and store nothing
                float a[kPerLane], b[kPerLane], o[kPerLane];
#pragma unroll
                for (int e = 0; e < kPerLane; ++e) {
                    a[e] = pa[e * kExprThreads];
                    b[e] = pb[e * kExprThreads];
                }
                apply(q, a, b, o, tabs);
#pragma unroll
                for (int e = 0; e < kPerLane; ++e) d[e * kExprThreads] = o[e];
            }
        }
    }
}

}  // namespace
}  // namespace ctamd

using namespace ctamd;

extern "C" int ctamd_expr_run_f32(const ctamd_expr_insn* prog, int n_insn, const float* const* inputs, int n_inputs,
                                  float* const* outputs, int n_outputs, int32_t* status, size_t rows, size_t cols,
                                  void* stream) {
    if (n_insn < 0 || n_inputs < 0 || n_outputs < 0) return fail(CTAMD_EINVAL, "%s: negative count", __func__);
    if (n_insn > kMaxInsns) return fail(CTAMD_ERANGE, "%s: more than %d instructions", __func__, kMaxInsns);
    if (n_inputs > kMaxPorts || n_outputs > kMaxPorts)
        return fail(CTAMD_ERANGE, "%s: more than %d inputs or outputs", __func__, kMaxPorts);
    if (n_insn && !prog) return fail(CTAMD_EINVAL, "%s: null program", __func__);
    const size_t total = rows * cols;
    if (cols && total / cols != rows) return fail(CTAMD_ERANGE, "%s: extent too large", __func__);
    if (cols > 0x3fffffffu) return fail(CTAMD_ERANGE, "%s: row too long", __func__);
    if (total == 0 || n_insn == 0) return CTAMD_OK;

    ExprArgs g;
    bool vec = (total % 4 == 0) && (cols % 4 == 0);
    for (int i = 0; i < n_inputs; ++i) {
        if (!inputs || !inputs[i]) return fail(CTAMD_EINVAL, "%s: null input %d", __func__, i);
        g.in[i] = inputs[i];
        vec = vec && aligned16(inputs[i]);
    }
    for (int i = 0; i < n_outputs; ++i) {
        if (!outputs || !outputs[i]) return fail(CTAMD_EINVAL, "%s: null output %d", __func__, i);
        g.out[i] = outputs[i];
        vec = vec && aligned16(outputs[i]);
    }
    // every slot must be written before it is read, every port must exist: a bad program must not
    // become a bad access on the device
    bool written[kMaxSlots] = {};
    int slots_used = 0;
    bool needs_status = false;
    double bytes = 0;
    for (int pc = 0; pc < n_insn; ++pc) {
        const ctamd_expr_insn& q = prog[pc];
        DevInsn& d = g.prog[pc];
        d.op = q.op; d.dst = q.dst; d.a = q.a; d.b = q.b; d.imm = q.imm;
        d.rcp = (q.op == CTAMD_EX_DIVS) ? 1.0 / double(q.imm) : 0.0;
        auto slot_ok = [&](int s) { return s < kMaxSlots && written[s]; };
        switch (q.op) {
            case CTAMD_EX_LOAD_FULL:
            case CTAMD_EX_LOAD_ROW:
                if (q.a >= n_inputs) return fail(CTAMD_EINVAL, "%s: instruction %d loads input %d of %d", __func__, pc, q.a, n_inputs);
                if (q.dst >= kMaxSlots) return fail(CTAMD_ERANGE, "%s: instruction %d writes slot %d", __func__, pc, q.dst);
                d.b = 0;
                bytes += (q.op == CTAMD_EX_LOAD_FULL) ? 4.0 * double(total) : 4.0 * double(cols);
                break;
            case CTAMD_EX_STORE:
            case CTAMD_EX_STORE_ZP:
                if (q.dst >= n_outputs) return fail(CTAMD_EINVAL, "%s: instruction %d stores output %d of %d", __func__, pc, q.dst, n_outputs);
                if (!slot_ok(q.a)) return fail(CTAMD_EINVAL, "%s: instruction %d reads an unwritten slot", __func__, pc);
                d.b = q.a;
                bytes += 4.0 * double(total);
                break;
            case CTAMD_EX_DIVCHK:
                if (!slot_ok(q.a)) return fail(CTAMD_EINVAL, "%s: instruction %d reads an unwritten slot", __func__, pc);
                d.b = q.a; d.dst = q.a;
                needs_status = true;
                break;
            case CTAMD_EX_ADD: case CTAMD_EX_SUB: case CTAMD_EX_MUL: case CTAMD_EX_DIV: case CTAMD_EX_RELUMUL:
                if (!slot_ok(q.a) || !slot_ok(q.b)) return fail(CTAMD_EINVAL, "%s: instruction %d reads an unwritten slot", __func__, pc);
                if (q.dst >= kMaxSlots) return fail(CTAMD_ERANGE, "%s: instruction %d writes slot %d", __func__, pc, q.dst);
                break;
            case CTAMD_EX_NEG: case CTAMD_EX_RELU: case CTAMD_EX_SIGMOID: case CTAMD_EX_TANH: case CTAMD_EX_SIN:
            case CTAMD_EX_COS: case CTAMD_EX_ADDS: case CTAMD_EX_MULS: case CTAMD_EX_DIVS: case CTAMD_EX_RSUBS:
                if (!slot_ok(q.a)) return fail(CTAMD_EINVAL, "%s: instruction %d reads an unwritten slot", __func__, pc);
                if (q.dst >= kMaxSlots) return fail(CTAMD_ERANGE, "%s: instruction %d writes slot %d", __func__, pc, q.dst);
                d.b = q.a;
                break;
            default:
                return fail(CTAMD_EINVAL, "%s: instruction %d has unknown operator %d", __func__, pc, q.op);
        }
        if (q.op != CTAMD_EX_STORE && q.op != CTAMD_EX_STORE_ZP && q.op != CTAMD_EX_DIVCHK) {
            written[q.dst] = true;
            if (q.dst + 1 > slots_used) slots_used = q.dst + 1;
        }
    }
    if (needs_status && !status) return fail(CTAMD_EINVAL, "%s: the program checks divisors but status is null", __func__);
    g.status = status;
    g.total = total;
    g.cols = unsigned(cols);
    g.n_insn = n_insn;
    g.vec = vec ? 1 : 0;
    g.has_row = 0;
    for (int pc = 0; pc < n_insn; ++pc) g.has_row |= (prog[pc].op == CTAMD_EX_LOAD_ROW);
    if (slots_used < 1) slots_used = 1;

    const size_t lds = size_t(slots_used) * kPerLane * kExprThreads * sizeof(float);
    // more than the default 64 KiB of LDS per block has to be asked for, once per device
    static int lds_raised[kMaxDevices] = {};
    int dev = 0;
    if (lds > (size_t(60) << 10)) {
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(CTAMD_EHIP, "%s: no current device", __func__);
        if (!lds_raised[dev]) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(expr_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               int(size_t(kMaxSlots) * kPerLane * kExprThreads * sizeof(float)));
            if (e != hipSuccess) return fail(CTAMD_EHIP, "%s: %d value slots need %zu bytes of LDS: %s", __func__, slots_used, lds,
                                             hipGetErrorString(e));
            lds_raised[dev] = 1;
        }
    }
    const size_t per_pass = size_t(kExprThreads) * kPerLane;
    const size_t passes = (total + per_pass - 1) / per_pass;
    // resident blocks: LDS allows 160 KiB / lds per CU (at most 8 of 256 threads); more blocks than
    // that only queue, fewer passes than that leave CUs idle
    const int cus = compute_units() > 0 ? compute_units() : 256;
    size_t per_cu = (size_t(160) << 10) / (lds + 512);
    if (per_cu > 8) per_cu = 8;
    if (per_cu < 1) per_cu = 1;
    size_t blocks = size_t(cus) * per_cu;
    if (blocks > passes) blocks = passes;
    account(bytes, 0.0);
    hipLaunchKernelGGL(expr_kernel, dim3(unsigned(blocks)), dim3(kExprThreads), lds, as_stream(stream), g);
    return launched(__func__);
}
