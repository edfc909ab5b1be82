// Fused elementwise expressions: a straight-line program of the per-element operators (the same
// functors the one-operator kernels use) evaluated in ONE pass over memory - every input is read
// once, every output written once, intermediates never leave the chip.  The front-end compiles
// both an expression's forward values and its tape gradients into such programs, so a chain like
// Y = sigmoid(X / r) - tanh(X) * sin(X) + cos(-X) is one launch forward and one launch backward
// instead of nine and about fifteen, with the bits of the operator-by-operator evaluation in the
// exact math mode (a few ulp from them in the single-precision one).
//
// The kernel is an interpreter: the program sits in the kernel arguments (uniform, read through
// the scalar unit, one instruction ahead of its execution), so every instruction is a scalar branch
// to one functor's code, applied to the eight elements each lane owns (two 128-bit words; four
// where a program has too many values live for LDS).  The latest result stays in registers and the
// next instruction takes it from there; only a value that a later instruction needs goes to an LDS
// place - word t of place p belongs to lane t, consecutive lanes on consecutive words, no
// conflicts - and places are reused as values die.  A chain of cheap operators still pays about
// thirty scalar instructions of interpretation per operator, shared by eight elements; for the
// transcendental operators that is noise, and their arithmetic - not memory - bounds the kernel.
// (Registers cannot hold the places: the place number is data.)
#include "common.h"
#include "devmath.h"
#include "functors.h"
#include "expr_jit.h"

#include <cfloat>
#include <utility>

namespace ctamd {
namespace {

constexpr int kExprThreads = 256;
constexpr int kMaxHalves = 2;                 // 128-bit words per lane and pass: one or two
constexpr int kMaxInsns = CTAMD_EXPR_MAX_INSNS;
constexpr int kMaxSlots = CTAMD_EXPR_MAX_SLOTS;          // slot numbers a program may name
constexpr int kWordBytes = kExprThreads * 16;            // one value of a block in LDS, per 128-bit word of a lane
constexpr int kLdsBudget = 155 << 10;                    // for values (160 KiB less the tables)
constexpr int kMaxLive = kLdsBudget / kWordBytes;        // values that can be live in LDS at once, one word per lane
constexpr int kMaxPorts = CTAMD_EXPR_MAX_PORTS;
constexpr int kMaxDevices = 64;

// What the kernel runs: the caller's program after value numbering.  Every instruction's result
// stays in registers (the "carry") until the next result replaces it.  An instruction works in
// place on the carry: its operand a is the carry, fetched from LDS first where the carry holds
// something else (kAFetch); operand b is always fetched from LDS (kBFetch: for x * x the value is kept
// and fetched back); the result
// goes to LDS only if an instruction further on has to fetch it (kKeep).  Where only the second
// operand of a - b, a / b or the ReLU gradient is in the carry, the operands change places and the
// operator is one of the reversed ones below.  LDS places are handed out by liveness, so a program
// may name many slots and still occupy few.
enum : uint8_t { kAFetch = 1, kBFetch = 2, kKeep = 4 };
enum : uint8_t { kRevSub = 32, kRevDiv = 33, kRevReluMul = 34 };   // b - a, b / a, a * (b > 0 ? 1 : 0)
struct DevInsn {
    uint8_t op, flags;
    uint16_t dst;                             // LDS place of the result (kKeep; in 128-bit words of a one-word-per-lane layout); stores: output port
    uint16_t a, b;                            // LDS places of the operands; loads: a = input port
    union {
        float imm;
        double rcp;                           // DIVS: 1 / double(imm)
    };
};
static_assert(sizeof(DevInsn) == 16, "one 128-bit scalar load per instruction");

// An instruction as the kernel holds it: fetched with ONE 128-bit load through the scalar unit and
// taken apart with scalar bit operations.  (Read field by field, the 8- and 16-bit members came
// through the vector memory path: every fetch then waited on the vector memory counter, which also
// counts the loads issued a pass ahead.)
struct Insn {
    uint32_t op, flags, dst, a, b;
    float imm;
    double rcp;
};

constexpr int kWholeFetchInsns = 10;      // programs of this many instructions or more fetch them whole

struct alignas(16) ExprArgs {
    const float* in[kMaxPorts];
    float* out[kMaxPorts];
    int32_t* status;
    size_t total;                             // elements of a full-shape value
    unsigned cols;                            // row length (row-vector loads)
    int n_insn;
    int has_row;                              // the program loads a row vector
    int n_lead;                               // the first n_lead instructions are loads (at most kLeadLoads)
    int n_tail;                               // VEC: the last n_tail instructions are stores (at most kTailStores)
    alignas(16) DevInsn prog[kMaxInsns + 1];  // one spare: the kernel fetches an instruction ahead
};

// WHOLE: one 128-bit scalar load (long programs: 5% faster on the nine-operator expression);
// otherwise field by field, which leaves less scalar work per instruction and is what a program of
// a few cheap operators runs faster with (4%).
template <bool WHOLE>
__device__ __forceinline__ Insn fetch_insn(const ExprArgs& g, int pc) {
    Insn q;
    if (!WHOLE) {
        const DevInsn& d = g.prog[pc];
        q.op = d.op; q.flags = d.flags; q.dst = d.dst; q.a = d.a; q.b = d.b;
        q.imm = d.imm;
        q.rcp = d.rcp;
        return q;
    }
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const u4 w = *reinterpret_cast<const u4*>(&g.prog[pc]);
    q.op = w[0] & 0xffu;
    q.flags = (w[0] >> 8) & 0xffu;
    q.dst = w[0] >> 16;
    q.a = w[1] & 0xffffu;
    q.b = w[1] >> 16;
    q.imm = __uint_as_float(w[2]);
    q.rcp = __hiloint2double(int(w[3]), int(w[2]));
    return q;
}

// The second operand of a two-operand operator always comes from LDS, fetched (through `second`)
// inside the operator's own case: fetched ahead of the switch - or defaulted to the carry for
// x * x - it is a second live copy of eight registers at every operator, also the one-operand
// ones, and keeps the compiler from computing the result in the carry's own registers (a dozen
// register moves per operator on the nine-operator program).
template <bool FASTM, int N, class Second>
__device__ __forceinline__ void apply(const Insn& q, float (&c)[N], Second second, const Tables& t) {
    float b[N];
    switch (q.op) {
        case CTAMD_EX_ADD: second(b); each(c, [&](int e) { return c[e] + b[e]; }); break;
        case CTAMD_EX_SUB: second(b); each(c, [&](int e) { return c[e] - b[e]; }); break;
        case kRevSub: second(b); each(c, [&](int e) { return b[e] - c[e]; }); break;
        case CTAMD_EX_MUL: second(b); each(c, [&](int e) { return c[e] * b[e]; }); break;
        case CTAMD_EX_DIV: second(b); each(c, [&](int e) { return c[e] / b[e]; }); break;
        case kRevDiv: second(b); each(c, [&](int e) { return b[e] / c[e]; }); break;
        case CTAMD_EX_NEG: each(c, [&](int e) { return -c[e]; }); break;
        case CTAMD_EX_RELU: each(c, [&](int e) { return (0.0f < c[e]) ? c[e] : 0.0f; }); break;
        case CTAMD_EX_SIGMOID:
            if (FASTM) sigmoid_fast(c, t);
            else each(c, [&](int e) { return sigmoid_ref(c[e], t); });
            break;
        // tanh is the reference's (e^x - e^-x) / (e^x + e^-x) on glibc's own floats in both modes: near
        // zero that quotient follows the rounding errors of the two exponentials, so nothing short
        // of their exact bits stays within 2 ulp of it
        case CTAMD_EX_TANH: each(c, [&](int e) { return tanh_ref(c[e], t); }); break;
        case CTAMD_EX_SIN: sin_or_cos<FASTM, 0>(c, t); break;       // two cases: the compiler then knows which of the two it builds
        case CTAMD_EX_COS: sin_or_cos<FASTM, 1>(c, t); break;
        case CTAMD_EX_ADDS: each(c, [&](int e) { return c[e] + q.imm; }); break;
        case CTAMD_EX_MULS: each(c, [&](int e) { return c[e] * q.imm; }); break;
        case CTAMD_EX_DIVS: each(c, [&](int e) { return cta_div_rcp(c[e], q.rcp); }); break;
        case CTAMD_EX_RSUBS: each(c, [&](int e) { return q.imm - c[e]; }); break;
        case CTAMD_EX_RELUMUL: second(b); each(c, [&](int e) { return b[e] * ((c[e] > 0.0f) ? 1.0f : 0.0f); }); break;
        case kRevReluMul: second(b); each(c, [&](int e) { return c[e] * ((b[e] > 0.0f) ? 1.0f : 0.0f); }); break;
        default: break;
    }
}

constexpr int kLeadLoads = 3;   // loads at the head of a program that run one pass ahead
constexpr int kTailStores = 2;  // stores at the end of a program that are issued one pass late (VEC only)

template <int H>
struct Vals {
    v4f h[H];
};

// Where a lane's 4 H elements of one pass live.  VEC: H 128-bit words 256 words apart (all
// pointers 16-byte aligned, total and cols multiples of four, fewer than 2^32 words): word index
// of the first, and for row vectors the word indices within the row, stepped from pass to pass
// without a division.  Otherwise: elements 256 apart, 32-bit accesses, any shape.
template <bool VEC, int H>
struct Place {
    size_t first;            // VEC: word index of word 0; else: element index of element 0
    unsigned col[H];         // VEC: word index within the row of each word; else unused
};

template <bool VEC, int H>
__device__ __forceinline__ Vals<H> load_elements(const ExprArgs& g, const Insn& q, const Place<VEC, H>& at) {
    const float* __restrict__ src = g.in[q.a];
    const bool row = (q.op == CTAMD_EX_LOAD_ROW);
    Vals<H> v;
#pragma unroll
    for (int h = 0; h < H; ++h) v.h[h] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    if (VEC) {
        // One load with the streaming hint for both kinds of operand.  Written as a hinted load of
        // a full tensor and a plain one of a row vector, the compiler folds the two into ONE plain
        // load of a selected address, and the operands lose their hint: with two inputs of 256 MiB
        // each, a + b then takes 148 instead of 139 us and relu(a * b + 5) 139 instead of 130 us.
        // Kept apart as two loads under a branch they cost more than that gains (the nine-operator
        // program: 236 against 223 us).  A row vector is small enough to be found in L2 again
        // whatever its hint says.
#pragma unroll
        for (int h = 0; h < H; ++h) {
            const size_t w = at.first + size_t(h) * kExprThreads;
            if (w < g.total / 4)
                v.h[h] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src) + (row ? size_t(at.col[h]) : w));
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4 * H; ++e) {
            size_t i = at.first + size_t(e) * kExprThreads;
            if (i < g.total) v.h[e / 4][e % 4] = src[row ? i % g.cols : i];
        }
    }
    return v;
}

template <bool VEC, bool FASTM, int H, bool WHOLE>
__global__ __launch_bounds__(kExprThreads, FASTM ? 4 : 3) void expr_kernel(ExprArgs g) {
    constexpr int N = 4 * H;                  // elements per lane and pass
    extern __shared__ v4f slots[];            // [places used][H][kExprThreads] 128-bit words
    __shared__ uint64_t s_exp2[32];
    __shared__ uint32_t s_pio4[24];
    stage_tables(s_exp2, s_pio4);
    const Tables tabs{s_exp2, s_pio4};
    const unsigned tid = threadIdx.x;
    v4f* const lane = slots + tid;
    // a place is given in 128-bit words of a one-word-per-lane layout; H words per lane scale it
    auto get = [&](unsigned place) {
        Vals<H> v;
#pragma unroll
        for (int h = 0; h < H; ++h) v.h[h] = lane[place * H + unsigned(h) * kExprThreads];
        return v;
    };
    auto put = [&](unsigned place, const Vals<H>& v) {
#pragma unroll
        for (int h = 0; h < H; ++h) lane[place * H + unsigned(h) * kExprThreads] = v.h[h];
    };
    const size_t per_pass = size_t(kExprThreads) * N;
    const size_t words_per_pass = size_t(kExprThreads) * H;
    const size_t passes = (g.total + per_pass - 1) / per_pass;

    Place<VEC, H> next;                        // of the pass whose head loads are issued next
    next.first = VEC ? size_t(blockIdx.x) * words_per_pass + tid : size_t(blockIdx.x) * per_pass + tid;
    const unsigned cols4 = g.cols / 4;
    const bool rows_used = VEC && g.has_row;
    const unsigned half_step = rows_used ? unsigned(kExprThreads % cols4) : 0u;
    const unsigned col_step = rows_used ? unsigned((size_t(gridDim.x) * words_per_pass) % cols4) : 0u;
    next.col[0] = rows_used ? unsigned(next.first % cols4) : 0u;
#pragma unroll
    for (int h = 1; h < H; ++h) {
        next.col[h] = next.col[h - 1] + half_step;
        if (rows_used && next.col[h] >= cols4) next.col[h] -= cols4;
    }
    auto advance = [&](Place<VEC, H>& p) {
        p.first += VEC ? size_t(gridDim.x) * words_per_pass : size_t(gridDim.x) * per_pass;
        if (rows_used) {
#pragma unroll
            for (int h = 0; h < H; ++h) {
                p.col[h] += col_step;
                if (p.col[h] >= cols4) p.col[h] -= cols4;
            }
        }
    };
    // The loads at the head of the program run one pass ahead, in registers: all of them go out
    // together, and they are in flight while the previous pass is being computed.
    Vals<H> pre[kLeadLoads];
    auto issue_lead = [&]() {
#pragma unroll
        for (int k = 0; k < kLeadLoads; ++k)
            if (k < g.n_lead) pre[k] = load_elements<VEC, H>(g, fetch_insn<WHOLE>(g, k), next);
    };
    // The stores at the end of the program go out one pass late, just before the next loads: the
    // memory counter of this hardware counts loads and stores in one order, so waiting for a
    // pass's loads would otherwise also wait for the stores of the pass before.
    Vals<H> post[kTailStores];
    size_t post_at = 0;
    bool post_full[H] = {};
    auto issue_tail = [&]() {
        if (VEC) {
#pragma unroll
            for (int k = 0; k < kTailStores; ++k)
                if (k < g.n_tail) {
                    v4f* __restrict__ dst = reinterpret_cast<v4f*>(g.out[fetch_insn<WHOLE>(g, g.n_insn - g.n_tail + k).dst]) + post_at;
#pragma unroll
                    for (int h = 0; h < H; ++h)
                        if (post_full[h]) __builtin_nontemporal_store(post[k].h[h], dst + h * kExprThreads);
                }
        }
    };
    auto zero_plus = [](Vals<H>& v) {
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) v.h[h][e] = 0.0f + v.h[h][e];
    };
    const int n_body = g.n_insn - (VEC ? g.n_tail : 0);
    Vals<H> carry;                             // the latest result
#pragma unroll
    for (int h = 0; h < H; ++h) carry.h[h] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    if (blockIdx.x < passes) issue_lead();
    for (size_t pass = blockIdx.x; pass < passes; pass += gridDim.x) {
        const Place<VEC, H> at = next;
        // one wait for this pass's loads on every path (vmcnt(0); 0x0F70 leaves the other counters
        // alone): with the waits only inside the conditional copies below, the compiler would
        // have to assume loads still in flight later on and wait again after the stores
        __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
        for (int k = 0; k < kLeadLoads; ++k)
            if (k < g.n_lead) put(fetch_insn<WHOLE>(g, k).dst, pre[k]);
        advance(next);
        issue_tail();
        if (pass + gridDim.x < passes) issue_lead();
        bool inside[H];
#pragma unroll
        for (int h = 0; h < H; ++h) inside[h] = VEC ? (at.first + size_t(h) * kExprThreads < g.total / 4) : true;
        Insn fetched = fetch_insn<WHOLE>(g, g.n_lead);    // instructions are fetched one ahead of their execution (the array has a spare entry)
        for (int pc = g.n_lead; pc < n_body; ++pc) {
            const Insn q = fetched;
            fetched = fetch_insn<WHOLE>(g, pc + 1);
            if (q.op == CTAMD_EX_LOAD_FULL || q.op == CTAMD_EX_LOAD_ROW) {
                carry = load_elements<VEC, H>(g, q, at);
            } else if (q.op == CTAMD_EX_STORE || q.op == CTAMD_EX_STORE_ZP) {
                float* __restrict__ dst = g.out[q.dst];
                Vals<H> v = carry;
                if (q.flags & kAFetch) v = get(q.a);
                if (q.op == CTAMD_EX_STORE_ZP) zero_plus(v);
                if (VEC) {
#pragma unroll
                    for (int h = 0; h < H; ++h)
                        if (inside[h]) __builtin_nontemporal_store(v.h[h], reinterpret_cast<v4f*>(dst) + at.first + h * kExprThreads);
                } else {
#pragma unroll
                    for (int e = 0; e < N; ++e) {
                        size_t i = at.first + size_t(e) * kExprThreads;
                        if (i < g.total) dst[i] = v.h[e / 4][e % 4];
                    }
                }
                continue;
            } else if (q.op == CTAMD_EX_DIVCHK) {
                // the tape refuses to differentiate a division whose divisor has an element with
                // |b| < FLT_EPSILON (the reference: src/AutoDiff.cpp:1267-1284); reported through status
                bool bad = false;
                Vals<H> v = carry;
                if (q.flags & kAFetch) v = get(q.a);
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    const bool live = VEC ? inside[e / 4] : (at.first + size_t(e) * kExprThreads < g.total);
                    if (live) bad = bad || (fabsf(v.h[e / 4][e % 4]) < FLT_EPSILON);
                }
                if (bad) atomicOr(g.status, 1);
                continue;
            } else {
                // lanes past the end compute on the zeros their loads gave them and store nothing
                if (q.flags & kAFetch) carry = get(q.a);
                float c[N];
#pragma unroll
                for (int e = 0; e < N; ++e) c[e] = carry.h[e / 4][e % 4];
                apply<FASTM, N>(q, c, [&](float (&b)[N]) {
                    const Vals<H> vb = get(q.b);
#pragma unroll
                    for (int e = 0; e < N; ++e) b[e] = vb.h[e / 4][e % 4];
                }, tabs);
#pragma unroll
                for (int e = 0; e < N; ++e) carry.h[e / 4][e % 4] = c[e];
            }
            if (q.flags & kKeep) put(q.dst, carry);
        }
        if (VEC) {
#pragma unroll
            for (int k = 0; k < kTailStores; ++k)
                if (k < g.n_tail) {
                    const Insn q = fetch_insn<WHOLE>(g, n_body + k);
                    Vals<H> v = carry;
                    if (q.flags & kAFetch) v = get(q.a);
                    if (q.op == CTAMD_EX_STORE_ZP) zero_plus(v);
                    post[k] = v;
                }
            post_at = at.first;
#pragma unroll
            for (int h = 0; h < H; ++h) post_full[h] = inside[h];
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
    bool needs_status = false;
    double bytes = 0;
    for (int pc = 0; pc < n_insn; ++pc) {
        const ctamd_expr_insn& q = prog[pc];
        DevInsn& d = g.prog[pc];
        d.op = q.op; d.flags = 0; d.dst = q.dst; d.a = q.a; d.b = q.b;
        d.rcp = 0.0;
        if (q.op == CTAMD_EX_DIVS) d.rcp = 1.0 / double(q.imm);
        else d.imm = q.imm;
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
        }
    }
    if (needs_status && !status) return fail(CTAMD_EINVAL, "%s: the program checks divisors but status is null", __func__);
    // a program that has been launched often enough runs as a kernel compiled for it
    {
        const int rc = jit_try_launch(prog, n_insn, inputs, n_inputs, outputs, n_outputs, status, rows, cols, vec, fast_math(), stream);
        if (rc != kJitDeclined) {
            if (rc == CTAMD_OK) account(bytes, 0.0);
            return rc;
        }
    }
    g.status = status;
    g.total = total;
    g.cols = unsigned(cols);
    g.n_insn = n_insn;
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

    // Value numbering.  The kernel keeps the latest result in registers; an operand produced by
    // the instruction that wrote those registers last is taken from there, every other operand
    // is fetched from LDS, so only results with such a reader are kept.  The loads at the head run
    // a pass ahead and are always kept.
    auto is_load = [](int op) { return op == CTAMD_EX_LOAD_FULL || op == CTAMD_EX_LOAD_ROW; };
    auto is_sink = [](int op) { return op == CTAMD_EX_STORE || op == CTAMD_EX_STORE_ZP || op == CTAMD_EX_DIVCHK; };
    auto is_binary = [](int op) { return (op >= CTAMD_EX_ADD && op <= CTAMD_EX_DIV) || op == CTAMD_EX_RELUMUL; };
    int producer[kMaxSlots];
    for (int& v : producer) v = -1;
    int from_a[kMaxInsns], from_b[kMaxInsns], last_fetch[kMaxInsns];
    bool kept[kMaxInsns];
    int in_carry = -1;
    for (int pc = 0; pc < n_insn; ++pc) {
        const ctamd_expr_insn& q = prog[pc];
        DevInsn& d = g.prog[pc];
        from_a[pc] = from_b[pc] = last_fetch[pc] = -1;
        kept[pc] = pc < g.n_lead;
        if (!is_load(q.op)) from_a[pc] = producer[q.a];
        if (is_binary(q.op)) {
            from_b[pc] = producer[q.b];
            if (from_a[pc] != in_carry && from_b[pc] == in_carry) {   // only b is in the carry: change places
                std::swap(from_a[pc], from_b[pc]);
                if (q.op == CTAMD_EX_SUB) d.op = kRevSub;
                if (q.op == CTAMD_EX_DIV) d.op = kRevDiv;
                if (q.op == CTAMD_EX_RELUMUL) d.op = kRevReluMul;
            }
        }
        auto fetch = [&](int from, uint8_t flag) {
            if (from < 0 || (from == in_carry && flag == kAFetch)) return;   // a second operand never comes from the carry (x * x: kept and fetched)
            d.flags |= flag;
            kept[from] = true;
            last_fetch[from] = pc;
        };
        fetch(from_a[pc], kAFetch);
        fetch(from_b[pc], kBFetch);
        if (!is_sink(q.op)) {
            producer[q.dst] = pc;
            if (pc >= g.n_lead) in_carry = pc;
        }
    }
    // LDS places by liveness: a place is free again after the last instruction that fetches it (the
    // result of that very instruction may take it: a lane reads its words before it writes them)
    int place[kMaxInsns];
    bool busy[kMaxLive] = {};
    int places_used = 0;
    for (int pc = 0; pc < n_insn; ++pc) {
        DevInsn& d = g.prog[pc];
        const int op = prog[pc].op;
        if (d.flags & kAFetch) d.a = uint16_t(place[from_a[pc]] * kExprThreads);
        if (d.flags & kBFetch) d.b = uint16_t(place[from_b[pc]] * kExprThreads);
        if ((d.flags & kAFetch) && last_fetch[from_a[pc]] == pc) busy[place[from_a[pc]]] = false;
        if ((d.flags & kBFetch) && last_fetch[from_b[pc]] == pc) busy[place[from_b[pc]]] = false;
        if (!is_sink(op) && kept[pc]) {
            int p = 0;
            while (p < kMaxLive && busy[p]) ++p;
            if (p == kMaxLive) return fail(CTAMD_ERANGE, "%s: more than %d values are live at instruction %d", __func__, kMaxLive, pc);
            busy[p] = true;
            place[pc] = p;
            if (p + 1 > places_used) places_used = p + 1;
            d.flags |= kKeep;
            d.dst = uint16_t(p * kExprThreads);
        }
        if (pc == g.n_lead - 1)                 // head loads nobody fetches: written at the start of a pass, free after
            for (int k = 0; k < g.n_lead; ++k)
                if (last_fetch[k] < 0) busy[place[k]] = false;
    }
    if (places_used < 1) places_used = 1;
    g.prog[n_insn] = g.prog[n_insn - 1];        // the spare entry: fetched, never run
    // Two 128-bit words per lane and pass halve the interpretation per element and double what a
    // wave has in flight; with seven or more values live, LDS would hold fewer than three such
    // blocks per CU, and one word per lane - twice the blocks - is faster (config-5 gradient program,
    // 8 values live: 227 against 246 us).
    const int words = (kLdsBudget / (places_used * kWordBytes * 2) >= 3) ? 2 : 1;

    const size_t lds = size_t(places_used) * kWordBytes * words;
    using Kernel = void (*)(ExprArgs);
    static const Kernel kernels[2][2][2][kMaxHalves] = {
        {{{expr_kernel<false, false, 1, false>, expr_kernel<false, false, 2, false>}, {expr_kernel<false, true, 1, false>, expr_kernel<false, true, 2, false>}},
         {{expr_kernel<true, false, 1, false>, expr_kernel<true, false, 2, false>}, {expr_kernel<true, true, 1, false>, expr_kernel<true, true, 2, false>}}},
        {{{expr_kernel<false, false, 1, true>, expr_kernel<false, false, 2, true>}, {expr_kernel<false, true, 1, true>, expr_kernel<false, true, 2, true>}},
         {{expr_kernel<true, false, 1, true>, expr_kernel<true, false, 2, true>}, {expr_kernel<true, true, 1, true>, expr_kernel<true, true, 2, true>}}}};
    const bool fastm = fast_math();
    const int whole = g.n_insn >= kWholeFetchInsns ? 1 : 0;
    const Kernel kernel = kernels[whole][vec ? 1 : 0][fastm ? 1 : 0][words - 1];
    // more than the default 64 KiB of LDS per block has to be asked for, once per device
    static int lds_raised[kMaxDevices] = {};
    int dev = 0;
    if (lds > (size_t(60) << 10)) {
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(CTAMD_EHIP, "%s: no current device", __func__);
        if (!lds_raised[dev]) {
            hipError_t e = hipSuccess;
            for (int i = 0; i < 2 * 2 * 2 * kMaxHalves; ++i)
                if (e == hipSuccess)
                    e = hipFuncSetAttribute(reinterpret_cast<const void*>((&kernels[0][0][0][0])[i]), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget);
            if (e != hipSuccess) return fail(CTAMD_EHIP, "%s: %d live values need %zu bytes of LDS: %s", __func__, places_used, lds,
                                             hipGetErrorString(e));
            lds_raised[dev] = 1;
        }
    }
    const size_t per_pass = size_t(kExprThreads) * 4 * words;
    const size_t passes = (total + per_pass - 1) / per_pass;
    // as many blocks as stay resident (registers and LDS decide; asked once per kernel and LDS
    // size): more would only queue behind them and break the one-pass-ahead loads, fewer leave CUs idle
    const int cus = compute_units() > 0 ? compute_units() : 256;
    static int resident[2][2][2][kMaxHalves][kMaxLive + 1] = {};
    int& per_cu_cached = resident[whole][vec ? 1 : 0][fastm ? 1 : 0][words - 1][places_used];
    if (per_cu_cached == 0) {
        int nb = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, reinterpret_cast<const void*>(kernel), kExprThreads, lds);
        if (e != hipSuccess || nb < 1) nb = 1;
        per_cu_cached = nb;
    }
    size_t per_cu = size_t(per_cu_cached);
    size_t blocks = size_t(cus) * per_cu;
    if (blocks > passes) blocks = passes;
    account(bytes, 0.0);
    hipLaunchKernelGGL(kernel, dim3(unsigned(blocks)), dim3(kExprThreads), lds, as_stream(stream), g);
    return launched(__func__);
}
