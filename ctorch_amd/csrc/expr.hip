// Fused elementwise expressions: a straight-line program of the per-element operators (the same
// functors the one-operator kernels use) evaluated in ONE pass over memory - every input is read
// once, every output written once, intermediates never leave the chip.  The front-end compiles
// both an expression's forward values and its tape gradients into such programs, so a chain like
// Y = sigmoid(X / r) - tanh(X) * sin(X) + cos(-X) is one launch forward and one launch backward
// instead of nine and about fifteen, with the bits of the operator-by-operator evaluation.
//
// The kernel is an interpreter: the program sits in the kernel arguments (uniform, read through
// the scalar unit), so every instruction is a scalar branch to one functor's code, applied to the
// four elements each lane owns.  Values live in LDS "slots": the four elements of lane t in slot s
// are the 128-bit word slots[s * 256 + t] - one LDS instruction per operand, consecutive lanes on
// consecutive words, no conflicts.  An instruction costs two 128-bit LDS reads and one write next
// to its arithmetic and about twenty scalar / address instructions of interpretation; for the
// transcendental operators that is noise, a chain of cheap operators pays it in full and still
// moves its bytes once instead of once per operator.  (Registers cannot hold the slots: the slot
// number is data.)
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
    int n_lead;                               // the first n_lead instructions are loads (at most kLeadLoads)
    int n_tail;                               // VEC: the last n_tail instructions are stores (at most kTailStores)
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

constexpr int kLeadLoads = 3;   // loads at the head of a program that run one pass ahead
constexpr int kTailStores = 2;  // stores at the end of a program that are issued one pass late (VEC only)

// Where a lane's four elements of one pass live.  VEC: four consecutive elements, one 128-bit
// access (all pointers 16-byte aligned, total and cols multiples of four, fewer than 2^32
// vectors): vector index v, and for row vectors the vector index within the row, stepped from
// pass to pass without a division.  Otherwise: elements 256 apart, 32-bit accesses, any shape.
template <bool VEC>
struct Place {
    size_t first;        // VEC: vector index; else: element index of element 0
    unsigned col;        // VEC: vector index within the row; else unused
};

template <bool VEC>
__device__ __forceinline__ v4f load_elements(const ExprArgs& g, const DevInsn& q, const Place<VEC>& at) {
    const float* __restrict__ src = g.in[q.a];
    const bool row = (q.op == CTAMD_EX_LOAD_ROW);
    v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (VEC) {
        // a full tensor is touched once (streaming hint); a row vector is re-read by every row and stays cached
        if (at.first < g.total / 4)
            v = row ? reinterpret_cast<const v4f*>(src)[at.col] : __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src) + at.first);
    } else {
#pragma unroll
        for (int e = 0; e < kPerLane; ++e) {
            size_t i = at.first + size_t(e) * kExprThreads;
            if (i < g.total) v[e] = src[row ? i % g.cols : i];
        }
    }
    return v;
}

template <bool VEC>
__global__ __launch_bounds__(kExprThreads) void expr_kernel(ExprArgs g) {
    extern __shared__ v4f slots[];            // [slots used][kExprThreads]: the four elements of a lane are one word
    __shared__ uint64_t s_exp2[32];
    __shared__ uint32_t s_pio4[24];
    stage_tables(s_exp2, s_pio4);
    const Tables tabs{s_exp2, s_pio4};
    const unsigned tid = threadIdx.x;
    const size_t per_pass = size_t(kExprThreads) * kPerLane;
    const size_t passes = (g.total + per_pass - 1) / per_pass;

    Place<VEC> next;                           // of the pass whose head loads are issued next
    next.first = VEC ? size_t(blockIdx.x) * kExprThreads + tid : size_t(blockIdx.x) * per_pass + tid;
    const unsigned cols4 = g.cols / 4;
    next.col = (VEC && g.has_row) ? unsigned(next.first % cols4) : 0u;
    const unsigned col_step = (VEC && g.has_row) ? unsigned((size_t(gridDim.x) * kExprThreads) % cols4) : 0u;
    auto advance = [&](Place<VEC>& p) {
        p.first += VEC ? size_t(gridDim.x) * kExprThreads : size_t(gridDim.x) * per_pass;
        if (VEC) {
            p.col += col_step;
            if (p.col >= cols4) p.col -= cols4;
        }
    };
    // The loads at the head of the program run one pass ahead, in registers: all of them go out
    // together, and they are in flight while the previous pass is being computed.
    v4f pre[kLeadLoads];
    auto issue_lead = [&]() {
#pragma unroll
        for (int k = 0; k < kLeadLoads; ++k)
            if (k < g.n_lead) pre[k] = load_elements<VEC>(g, g.prog[k], next);
    };
    // The stores at the end of the program go out one pass late, just before the next loads: the
    // memory counter of this hardware counts loads and stores in one order, so waiting for a
    // pass's loads would otherwise also wait for the stores of the pass before.
    v4f post[kTailStores];
    size_t post_at = 0;
    bool post_full = false;
    auto issue_tail = [&]() {
        if (VEC && post_full) {
#pragma unroll
            for (int k = 0; k < kTailStores; ++k)
                if (k < g.n_tail)
                    __builtin_nontemporal_store(post[k], reinterpret_cast<v4f*>(g.out[g.prog[g.n_insn - g.n_tail + k].dst]) + post_at);
        }
    };
    const int n_body = g.n_insn - (VEC ? g.n_tail : 0);
    if (blockIdx.x < passes) issue_lead();
    for (size_t pass = blockIdx.x; pass < passes; pass += gridDim.x) {
        const Place<VEC> at = next;
        // one wait for this pass's loads on every path (vmcnt(0); 0x0F70 leaves the other counters
        // alone): with the waits only inside the conditional copies below, the compiler would
        // have to assume loads still in flight later on and wait again after the stores
        __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
        for (int k = 0; k < kLeadLoads; ++k)
            if (k < g.n_lead) slots[unsigned(g.prog[k].dst) * kExprThreads + tid] = pre[k];
        advance(next);
        issue_tail();
        if (pass + gridDim.x < passes) issue_lead();
        const bool inside = VEC ? (at.first < g.total / 4) : true;
        for (int pc = g.n_lead; pc < n_body; ++pc) {
            const DevInsn q = g.prog[pc];
            v4f* __restrict__ d = slots + unsigned(q.dst) * kExprThreads + tid;
            const v4f* __restrict__ pa = slots + unsigned(q.a) * kExprThreads + tid;
            const v4f* __restrict__ pb = slots + unsigned(q.b) * kExprThreads + tid;
            if (q.op == CTAMD_EX_LOAD_FULL || q.op == CTAMD_EX_LOAD_ROW) {
                *d = load_elements<VEC>(g, q, at);
            } else if (q.op == CTAMD_EX_STORE || q.op == CTAMD_EX_STORE_ZP) {
                float* __restrict__ dst = g.out[q.dst];
                v4f v = *pa;
                if (q.op == CTAMD_EX_STORE_ZP) {
#pragma unroll
                    for (int e = 0; e < kPerLane; ++e) v[e] = 0.0f + v[e];
                }
                if (VEC) {
                    if (inside) __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(dst) + at.first);
                } else {
#pragma unroll
                    for (int e = 0; e < kPerLane; ++e) {
                        size_t i = at.first + size_t(e) * kExprThreads;
                        if (i < g.total) dst[i] = v[e];
                    }
                }
            } else if (q.op == CTAMD_EX_DIVCHK) {
                // the tape refuses to differentiate a division whose divisor has an element with
                // |b| < FLT_EPSILON (the reference: src/AutoDiff.cpp:1267-1284); reported through status
                bool bad = false;
                const v4f v = *pa;
#pragma unroll
                for (int e = 0; e < kPerLane; ++e) {
                    const bool live = VEC ? inside : (at.first + size_t(e) * kExprThreads < g.total);
                    if (live) bad = bad || (fabsf(v[e]) < FLT_EPSILON);
                }
                if (bad) atomicOr(g.status, 1);
            } else {
                // lanes past the end compute on the zeros their loads gave them and store nothing
                const v4f va = *pa, vb = *pb;
                float a[kPerLane], b[kPerLane], o[kPerLane];
#pragma unroll
                for (int e = 0; e < kPerLane; ++e) {
                    a[e] = va[e];
                    b[e] = vb[e];
                }
                apply(q, a, b, o, tabs);
                v4f vo;
#pragma unroll
                for (int e = 0; e < kPerLane; ++e) vo[e] = o[e];
                *d = vo;
            }
        }
        if (VEC) {
#pragma unroll
            for (int k = 0; k < kTailStores; ++k)
                if (k < g.n_tail) {
                    const DevInsn q = g.prog[n_body + k];
                    v4f v = slots[unsigned(q.a) * kExprThreads + tid];
                    if (q.op == CTAMD_EX_STORE_ZP) {
#pragma unroll
                        for (int e = 0; e < kPerLane; ++e) v[e] = 0.0f + v[e];
                    }
                    post[k] = v;
                }
            post_at = at.first;
            post_full = inside;
        }
    }
    issue_tail();
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
    bool vec = (total % 4 == 0) && (cols % 4 == 0) && (total / 4 <= 0xffffffffu);
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
    g.n_lead = 0;
    while (g.n_lead < n_insn && g.n_lead < kLeadLoads &&
           (prog[g.n_lead].op == CTAMD_EX_LOAD_FULL || prog[g.n_lead].op == CTAMD_EX_LOAD_ROW))
        ++g.n_lead;
    g.n_tail = 0;
    while (g.n_tail < kTailStores && g.n_lead + g.n_tail < n_insn &&
           (prog[n_insn - 1 - g.n_tail].op == CTAMD_EX_STORE || prog[n_insn - 1 - g.n_tail].op == CTAMD_EX_STORE_ZP))
        ++g.n_tail;
    if (slots_used < 1) slots_used = 1;

    const size_t lds = size_t(slots_used) * kPerLane * kExprThreads * sizeof(float);
    // more than the default 64 KiB of LDS per block has to be asked for, once per device
    static int lds_raised[kMaxDevices] = {};
    int dev = 0;
    if (lds > (size_t(60) << 10)) {
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(CTAMD_EHIP, "%s: no current device", __func__);
        if (!lds_raised[dev]) {
            const int most = int(size_t(kMaxSlots) * kPerLane * kExprThreads * sizeof(float));
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(expr_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, most);
            if (e == hipSuccess)
                e = hipFuncSetAttribute(reinterpret_cast<const void*>(expr_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, most);
            if (e != hipSuccess) return fail(CTAMD_EHIP, "%s: %d value slots need %zu bytes of LDS: %s", __func__, slots_used, lds,
                                             hipGetErrorString(e));
            lds_raised[dev] = 1;
        }
    }
    const size_t per_pass = size_t(kExprThreads) * kPerLane;
    const size_t passes = (total + per_pass - 1) / per_pass;
    // as many blocks as stay resident (registers and LDS decide; asked once per slot count): more
    // would only queue behind them and break the one-pass-ahead loads, fewer leave CUs idle
    const int cus = compute_units() > 0 ? compute_units() : 256;
    static int resident[2][kMaxSlots + 1] = {};
    int& per_cu_cached = resident[vec ? 1 : 0][slots_used];
    if (per_cu_cached == 0) {
        int nb = 0;
        hipError_t e = vec ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, expr_kernel<true>, kExprThreads, lds)
                           : hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, expr_kernel<false>, kExprThreads, lds);
        if (e != hipSuccess || nb < 1) nb = 1;
        per_cu_cached = nb;
    }
    size_t per_cu = size_t(per_cu_cached);
    size_t blocks = size_t(cus) * per_cu;
    if (blocks > passes) blocks = passes;
    account(bytes, 0.0);
    if (vec) hipLaunchKernelGGL(expr_kernel<true>, dim3(unsigned(blocks)), dim3(kExprThreads), lds, as_stream(stream), g);
    else hipLaunchKernelGGL(expr_kernel<false>, dim3(unsigned(blocks)), dim3(kExprThreads), lds, as_stream(stream), g);
    return launched(__func__);
}
