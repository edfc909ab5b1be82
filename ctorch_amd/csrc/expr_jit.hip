// Fused elementwise expressions compiled at run time.  The interpreter of expr.hip pays about twenty
// vector and thirty scalar instructions per operator for finding out what to do, and keeps its values
// in LDS because a place number is data.  A program that is launched again and again (a training
// step's expression and its gradient program) is instead written out as HIP source - one
// straight-line kernel whose values are registers - and compiled for the device with hiprtc, once per
// (program, math mode, access pattern), then kept for the life of the process.  The per-element
// arithmetic is the very text the interpreter is built from (devmath.h, expr_ops.h, embedded in this
// library at build time), compiled with the same contraction and packed-arithmetic flags, so both
// evaluators return the same bits.
//
// Two access patterns:
//   linear   a block owns 256 * V consecutive 128-bit words, one trip, all loads first;
//   columns  (programs with row-vector operands, rows of at least 128 words) a thread owns V words
//            of the row and walks a run of rows, next row's loads in flight while it computes.
//            Whatever depends on row vectors alone is computed once per thread, before the walk,
//            and a division by such a value becomes a multiplication by its double-precision
//            reciprocal (cta_div_rcp: the IEEE quotient, three instructions instead of twelve).
// Anything else - unaligned operands, ragged rows, short rows with row vectors - stays with the
// interpreter, as does a program until it has been launched `threshold` times (ctamd_set_expr_jit).
#include "expr_jit.h"

#include <hip/hiprtc.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace ctamd {
namespace {

// devmath.h and expr_ops.h as one string (build/jit_text.inc is written by ctorch_amd/build.py from
// those two files, their #include lines removed)
const char kDeviceText[] =
#include "jit_text.inc"
    ;

constexpr int kThreads = 256;
constexpr int kMaxDevices = 64;

std::atomic<int> g_threshold{2};
std::atomic<uint64_t> g_compiled{0}, g_jit_launches{0}, g_interp_launches{0}, g_failed{0};

struct JitArgs {                      // the compiled kernels' one argument; the text below declares the same
    const float* in[CTAMD_EXPR_MAX_PORTS];
    float* out[CTAMD_EXPR_MAX_PORTS];
    int32_t* status;
    unsigned long long total4;        // 128-bit words of a full-shape value
    unsigned cols4;                   // words of a row
    unsigned rows;
    unsigned rows_per_block;
};

struct Entry {
    int seen = 0;                     // launches so far
    bool tried = false, ok = false;
    int words = 1;                    // V
    bool columns = false;
    std::vector<char> code;
    hipModule_t module[kMaxDevices] = {};
    hipFunction_t fn[kMaxDevices] = {};
    int per_cu[kMaxDevices] = {};
};

std::mutex g_mu;
std::map<std::string, Entry> g_cache;

bool is_load(int op) { return op == CTAMD_EX_LOAD_FULL || op == CTAMD_EX_LOAD_ROW; }
bool is_sink(int op) { return op == CTAMD_EX_STORE || op == CTAMD_EX_STORE_ZP || op == CTAMD_EX_DIVCHK; }
bool is_binary(int op) { return (op >= CTAMD_EX_ADD && op <= CTAMD_EX_DIV) || op == CTAMD_EX_RELUMUL; }
bool is_transcendental(int op) { return op == CTAMD_EX_SIGMOID || op == CTAMD_EX_TANH || op == CTAMD_EX_SIN || op == CTAMD_EX_COS; }

std::string f32_literal(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    char buf[48];
    std::snprintf(buf, sizeof buf, "__uint_as_float(0x%08xu)", u);
    return buf;
}
std::string f64_literal(double v) {
    uint64_t u;
    std::memcpy(&u, &v, 8);
    char buf[64];
    std::snprintf(buf, sizeof buf, "__longlong_as_double(0x%016llxLL)", (unsigned long long)u);
    return buf;
}

// The program as single-assignment values: value pc is the result of instruction pc.
struct Ssa {
    std::vector<int> a, b;            // operand values of instruction pc (-1: none)
    std::vector<bool> inv;            // depends on row vectors (and constants) alone
    std::vector<bool> rcp;            // an invariant value some division by a varying value divides by
    bool valid = true;                // every operand was written before it is read
};

Ssa analyse(const ctamd_expr_insn* prog, int n, bool columns) {
    Ssa s;
    s.a.assign(size_t(n), -1);
    s.b.assign(size_t(n), -1);
    s.inv.assign(size_t(n), false);
    s.rcp.assign(size_t(n), false);
    int cur[CTAMD_EXPR_MAX_SLOTS];
    for (int& c : cur) c = -1;
    for (int pc = 0; pc < n; ++pc) {
        const ctamd_expr_insn& q = prog[pc];
        if (is_load(q.op)) {
            if (q.dst >= CTAMD_EXPR_MAX_SLOTS) {
                s.valid = false;
                return s;
            }
            s.inv[size_t(pc)] = columns && q.op == CTAMD_EX_LOAD_ROW;
            cur[q.dst] = pc;
            continue;
        }
        if (q.a >= CTAMD_EXPR_MAX_SLOTS || cur[q.a] < 0 || (is_binary(q.op) && (q.b >= CTAMD_EXPR_MAX_SLOTS || cur[q.b] < 0))) {
            s.valid = false;
            return s;
        }
        s.a[size_t(pc)] = cur[q.a];
        if (is_binary(q.op)) s.b[size_t(pc)] = cur[q.b];
        if (is_sink(q.op)) continue;
        if (q.dst >= CTAMD_EXPR_MAX_SLOTS) {
            s.valid = false;
            return s;
        }
        bool inv = s.inv[size_t(s.a[size_t(pc)])];
        if (is_binary(q.op)) inv = inv && s.inv[size_t(s.b[size_t(pc)])];
        s.inv[size_t(pc)] = inv;
        if (q.op == CTAMD_EX_DIV && !inv && s.inv[size_t(s.b[size_t(pc)])]) s.rcp[size_t(s.b[size_t(pc)])] = true;
        cur[q.dst] = pc;
    }
    return s;
}

std::string name(int v) { return "v" + std::to_string(v); }

// One instruction over the N elements of a lane.  `pre`: the invariant part (computed before the walk).
void emit_op(std::string& o, const ctamd_expr_insn* prog, const Ssa& s, int pc, bool fastm, bool in_columns_walk) {
    const ctamd_expr_insn& q = prog[pc];
    const std::string d = name(pc), a = name(s.a[size_t(pc)]);
    const std::string b = s.b[size_t(pc)] >= 0 ? name(s.b[size_t(pc)]) : std::string();
    auto loop = [&](const std::string& expr) {
        o += "    float " + d + "[N];\n    _Pragma(\"unroll\") for (int e = 0; e < N; ++e) " + d + "[e] = " + expr + ";\n";
    };
    auto in_place = [&](const std::string& call) {
        o += "    float " + d + "[N];\n    _Pragma(\"unroll\") for (int e = 0; e < N; ++e) " + d + "[e] = " + a + "[e];\n    " + call + ";\n";
    };
    switch (q.op) {
        case CTAMD_EX_ADD: loop(a + "[e] + " + b + "[e]"); break;
        case CTAMD_EX_SUB: loop(a + "[e] - " + b + "[e]"); break;
        case CTAMD_EX_MUL: loop(a + "[e] * " + b + "[e]"); break;
        case CTAMD_EX_DIV:
            if (in_columns_walk && s.inv[size_t(s.b[size_t(pc)])]) loop("cta_div_rcp(" + a + "[e], q" + std::to_string(s.b[size_t(pc)]) + "[e])");
            else loop(a + "[e] / " + b + "[e]");
            break;
        case CTAMD_EX_NEG: loop("-" + a + "[e]"); break;
        case CTAMD_EX_RELU: loop("(0.0f < " + a + "[e]) ? " + a + "[e] : 0.0f"); break;
        case CTAMD_EX_SIGMOID:
            if (fastm) in_place("sigmoid_fast(" + d + ", tabs)");
            else loop("sigmoid_ref(" + a + "[e], tabs)");
            break;
        case CTAMD_EX_TANH: loop("tanh_ref(" + a + "[e], tabs)"); break;
        case CTAMD_EX_SIN:
        case CTAMD_EX_COS: {
            // The single-precision routines of the default mode are exactly odd / even, so the sine or cosine
            // of a negated value is formed from the value itself: sin(x) and cos(-x) of one expression then
            // share their argument reduction and both polynomials (the compiler merges the equal work).
            // The bits are those of the operator applied to the negated value, which the interpreter forms.
            int src = s.a[size_t(pc)];
            bool flipped = false;
            while (fastm && prog[src].op == CTAMD_EX_NEG) {
                src = s.a[size_t(src)];
                flipped = !flipped;
            }
            const bool sine = q.op == CTAMD_EX_SIN;
            o += "    float " + d + "[N];\n    _Pragma(\"unroll\") for (int e = 0; e < N; ++e) " + d + "[e] = " + name(src) + "[e];\n    sin_or_cos<" +
                 (fastm ? "true" : "false") + ", " + (sine ? "0" : "1") + ">(" + d + ", tabs);\n";
            if (sine && flipped) o += "    _Pragma(\"unroll\") for (int e = 0; e < N; ++e) " + d + "[e] = -" + d + "[e];\n";
            break;
        }
        case CTAMD_EX_ADDS: loop(a + "[e] + " + f32_literal(q.imm)); break;
        case CTAMD_EX_MULS: loop(a + "[e] * " + f32_literal(q.imm)); break;
        case CTAMD_EX_DIVS: loop("cta_div_rcp(" + a + "[e], " + f64_literal(1.0 / double(q.imm)) + ")"); break;
        case CTAMD_EX_RSUBS: loop(f32_literal(q.imm) + " - " + a + "[e]"); break;
        case CTAMD_EX_RELUMUL: loop(b + "[e] * ((" + a + "[e] > 0.0f) ? 1.0f : 0.0f)"); break;
        default: break;
    }
}

// The kernel's source.  V: 128-bit words per lane (and row, in the columns pattern).
std::string generate(const ctamd_expr_insn* prog, int n, bool fastm, bool columns, int V) {
    const Ssa s = analyse(prog, n, columns);
    if (!s.valid) return std::string();
    bool tables = false;
    for (int pc = 0; pc < n; ++pc) tables = tables || is_transcendental(prog[pc].op);
    std::string o;
    o.reserve(1 << 16);
    o += "typedef unsigned int uint32_t;\ntypedef int int32_t;\ntypedef unsigned long long uint64_t;\ntypedef long long int64_t;\n"
         "#define __HIPCC__ 1\n";
    o += kDeviceText;
    o += "\nstruct JitArgs { const float* in[" + std::to_string(CTAMD_EXPR_MAX_PORTS) + "]; float* out[" + std::to_string(CTAMD_EXPR_MAX_PORTS) +
         "]; int* status; unsigned long long total4; unsigned cols4; unsigned rows; unsigned rows_per_block; };\n";
    o += "constexpr int V = " + std::to_string(V) + ";\nconstexpr int N = 4 * V;\n";
    o += "extern \"C\" __global__ __launch_bounds__(256) void expr_jit(JitArgs g) {\n";
    if (tables) {
        o += "    __shared__ uint64_t s_exp2[32];\n    __shared__ uint32_t s_pio4[24];\n    stage_tables(s_exp2, s_pio4);\n"
             "    const Tables tabs{s_exp2, s_pio4, nullptr};\n";
    }
    auto unpack = [&](int pc, const std::string& words) {
        o += "    float " + name(pc) + "[N];\n    _Pragma(\"unroll\") for (int e = 0; e < N; ++e) " + name(pc) + "[e] = " + words + "[e / 4][e % 4];\n";
    };
    auto store = [&](int pc, const std::string& index, const std::string& ok) {
        const ctamd_expr_insn& q = prog[pc];
        const std::string v = name(s.a[size_t(pc)]);
        const std::string zp = q.op == CTAMD_EX_STORE_ZP ? "0.0f + " : "";
        o += "    _Pragma(\"unroll\") for (int h = 0; h < V; ++h) if (" + ok + ") {\n        v4f w = {" + zp + v + "[4 * h], " + zp + v + "[4 * h + 1], " + zp + v +
             "[4 * h + 2], " + zp + v + "[4 * h + 3]};\n        __builtin_nontemporal_store(w, reinterpret_cast<v4f*>(g.out[" + std::to_string(q.dst) + "]) + " +
             index + ");\n    }\n";
    };
    auto divchk = [&](int pc, const std::string& ok) {
        const std::string v = name(s.a[size_t(pc)]);
        o += "    {\n        bool bad = false;\n        _Pragma(\"unroll\") for (int e = 0; e < N; ++e) { const int h = e / 4; bad = bad || ((" + ok + ") && __builtin_fabsf(" + v +
             "[e]) < 0x1p-23f); }\n        if (bad) atomicOr(g.status, 1);\n    }\n";
    };
    if (!columns) {
        o += "    const unsigned long long w0 = (unsigned long long)blockIdx.x * (256u * V) + threadIdx.x;\n"
             "    bool ok[V];\n    _Pragma(\"unroll\") for (int h = 0; h < V; ++h) ok[h] = w0 + h * 256u < g.total4;\n";
        // every load first, so that a lane has all its requests in flight before the first use
        for (int pc = 0; pc < n; ++pc) {
            if (!is_load(prog[pc].op)) continue;
            const std::string p = std::to_string(prog[pc].a);
            const std::string idx = prog[pc].op == CTAMD_EX_LOAD_ROW ? "(unsigned)(w0 + h * 256u) % g.cols4" : "w0 + h * 256u";
            o += "    v4f L" + std::to_string(pc) + "[V];\n    _Pragma(\"unroll\") for (int h = 0; h < V; ++h) L" + std::to_string(pc) +
                 "[h] = ok[h] ? __builtin_nontemporal_load(reinterpret_cast<const v4f*>(g.in[" + p + "]) + (" + idx + ")) : v4f{0.0f, 0.0f, 0.0f, 0.0f};\n";
        }
        for (int pc = 0; pc < n; ++pc) {
            const int op = prog[pc].op;
            if (is_load(op)) unpack(pc, "L" + std::to_string(pc));
            else if (op == CTAMD_EX_STORE || op == CTAMD_EX_STORE_ZP) store(pc, "w0 + h * 256u", "ok[h]");
            else if (op == CTAMD_EX_DIVCHK) divchk(pc, "ok[h]");
            else emit_op(o, prog, s, pc, fastm, false);
        }
        o += "}\n";
        return o;
    }
    // columns: the invariant part first
    o += "    const unsigned c0 = blockIdx.x * (256u * V) + threadIdx.x;\n"
         "    bool ok[V];\n    _Pragma(\"unroll\") for (int h = 0; h < V; ++h) ok[h] = c0 + h * 256u < g.cols4;\n"
         "    const unsigned r0 = blockIdx.y * g.rows_per_block;\n"
         "    const unsigned r1 = (g.rows - r0 < g.rows_per_block) ? g.rows : r0 + g.rows_per_block;\n";
    for (int pc = 0; pc < n; ++pc) {
        const int op = prog[pc].op;
        if (op == CTAMD_EX_LOAD_ROW) {
            o += "    v4f L" + std::to_string(pc) + "[V];\n    _Pragma(\"unroll\") for (int h = 0; h < V; ++h) L" + std::to_string(pc) +
                 "[h] = ok[h] ? reinterpret_cast<const v4f*>(g.in[" + std::to_string(prog[pc].a) + "])[c0 + h * 256u] : v4f{0.0f, 0.0f, 0.0f, 0.0f};\n";
            unpack(pc, "L" + std::to_string(pc));
        } else if (op == CTAMD_EX_DIVCHK && s.inv[size_t(s.a[size_t(pc)])]) {
            divchk(pc, "ok[h] && r0 < r1");
        } else if (!is_load(op) && !is_sink(op) && s.inv[size_t(pc)]) {
            emit_op(o, prog, s, pc, fastm, false);
        } else {
            continue;
        }
        if (!is_sink(op) && s.rcp[size_t(pc)])
            o += "    double q" + std::to_string(pc) + "[N];\n    _Pragma(\"unroll\") for (int e = 0; e < N; ++e) q" + std::to_string(pc) + "[e] = 1.0 / (double)" +
                 name(pc) + "[e];\n";
    }
    // the walk over the rows, the next row's loads one row ahead
    std::vector<int> full;
    for (int pc = 0; pc < n; ++pc)
        if (prog[pc].op == CTAMD_EX_LOAD_FULL) full.push_back(pc);
    auto issue = [&](const std::string& dst, const std::string& row) {
        for (int pc : full)
            o += "        _Pragma(\"unroll\") for (int h = 0; h < V; ++h) if (ok[h]) " + dst + std::to_string(pc) +
                 "[h] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(g.in[" + std::to_string(prog[pc].a) + "]) + ((unsigned long long)(" + row +
                 ") * g.cols4 + c0 + h * 256u));\n";
    };
    for (int pc : full)
        o += "    v4f X" + std::to_string(pc) + "[V];\n    _Pragma(\"unroll\") for (int h = 0; h < V; ++h) X" + std::to_string(pc) + "[h] = v4f{0.0f, 0.0f, 0.0f, 0.0f};\n";
    o += "    if (r0 < r1) {\n";
    issue("X", "r0");
    o += "    }\n    for (unsigned r = r0; r < r1; ++r) {\n";
    for (int pc : full)
        o += "    v4f L" + std::to_string(pc) + "[V];\n    _Pragma(\"unroll\") for (int h = 0; h < V; ++h) L" + std::to_string(pc) + "[h] = X" + std::to_string(pc) + "[h];\n";
    o += "    if (r + 1 < r1) {\n";
    issue("X", "r + 1");
    o += "    }\n    const unsigned long long at = (unsigned long long)r * g.cols4 + c0;\n";
    for (int pc = 0; pc < n; ++pc) {
        const int op = prog[pc].op;
        if (op == CTAMD_EX_LOAD_FULL) unpack(pc, "L" + std::to_string(pc));
        else if (op == CTAMD_EX_LOAD_ROW) continue;
        else if (op == CTAMD_EX_STORE || op == CTAMD_EX_STORE_ZP) store(pc, "at + h * 256u", "ok[h]");
        else if (op == CTAMD_EX_DIVCHK) { if (!s.inv[size_t(s.a[size_t(pc)])]) divchk(pc, "ok[h]"); }
        else if (!s.inv[size_t(pc)]) emit_op(o, prog, s, pc, fastm, true);
    }
    o += "    }\n}\n";
    return o;
}

bool compile(const std::string& src, std::vector<char>& code, std::string& log) {
    hiprtcProgram p;
    if (hiprtcCreateProgram(&p, src.c_str(), "ctamd_expr_jit.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
        log = "hiprtcCreateProgram failed";
        return false;
    }
    // the flags of the library's own build (ctorch_amd/build.py): no contraction, no packed fp32 arithmetic
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
                          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const hiprtcResult r = hiprtcCompileProgram(p, int(sizeof opts / sizeof opts[0]), opts);
    size_t n = 0;
    if (r != HIPRTC_SUCCESS) {
        if (hiprtcGetProgramLogSize(p, &n) == HIPRTC_SUCCESS && n > 1) {
            log.resize(n);
            hiprtcGetProgramLog(p, &log[0]);
        } else {
            log = hiprtcGetErrorString(r);
        }
        hiprtcDestroyProgram(&p);
        return false;
    }
    bool ok = hiprtcGetCodeSize(p, &n) == HIPRTC_SUCCESS && n > 0;
    if (ok) {
        code.resize(n);
        ok = hiprtcGetCode(p, code.data()) == HIPRTC_SUCCESS;
    }
    hiprtcDestroyProgram(&p);
    if (!ok) log = "hiprtcGetCode failed";
    return ok;
}

int env_int(const char* name_, int fallback) {
    const char* v = std::getenv(name_);
    return (v && *v) ? std::atoi(v) : fallback;
}

}  // namespace

int jit_try_launch(const ctamd_expr_insn* prog, int n_insn, const float* const* inputs, int n_inputs, float* const* outputs, int n_outputs,
                   int32_t* status, size_t rows, size_t cols, bool aligned, bool fastm, void* stream) {
    const int threshold = g_threshold.load(std::memory_order_relaxed);
    const auto declined = [&]() {
        g_interp_launches.fetch_add(1, std::memory_order_relaxed);
        return kJitDeclined;
    };
    if (threshold <= 0 || !aligned) return declined();
    const size_t total = rows * cols;
    bool has_row = false;
    int heavy = 0;
    for (int pc = 0; pc < n_insn; ++pc) {
        has_row = has_row || prog[pc].op == CTAMD_EX_LOAD_ROW;
        heavy += is_transcendental(prog[pc].op) ? 1 : 0;
    }
    const size_t cols4 = cols / 4;
    const bool columns = has_row;
    if (columns && (cols4 < 128 || rows > 0xffffffffu)) return declined();
    int words = heavy >= 3 ? 1 : 2;
    if (!columns && heavy == 0) words = 4;
    const int forced = env_int("CTAMD_JIT_WORDS", 0);
    if (forced == 1 || forced == 2 || forced == 4) words = forced;

    std::string key(reinterpret_cast<const char*>(prog), size_t(n_insn) * sizeof(ctamd_expr_insn));
    key.push_back(char(fastm ? 1 : 0));
    key.push_back(char(columns ? 1 : 0));
    key.push_back(char(words));

    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return declined();
    hipFunction_t fn = nullptr;
    int per_cu = 0;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        Entry& e = g_cache[key];
        ++e.seen;
        if (!e.tried) {
            if (e.seen < threshold) return declined();
            // never compile or load a module while the stream records a graph: the next eager launch does it
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(as_stream(stream), &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return declined();
            e.tried = true;
            e.words = words;
            e.columns = columns;
            std::string log;
            const std::string src = generate(prog, n_insn, fastm, columns, words);
            e.ok = compile(src, e.code, log);
            if (!e.ok) {
                g_failed.fetch_add(1, std::memory_order_relaxed);
                if (env_int("CTAMD_JIT_VERBOSE", 0)) std::fprintf(stderr, "ctorch_amd: run-time compilation of a fused expression failed, the interpreter runs it:\n%s\n", log.c_str());
            } else {
                g_compiled.fetch_add(1, std::memory_order_relaxed);
            }
        }
        if (!e.ok) return declined();
        if (!e.fn[dev]) {
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(as_stream(stream), &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return declined();
            if (hipModuleLoadData(&e.module[dev], e.code.data()) != hipSuccess ||
                hipModuleGetFunction(&e.fn[dev], e.module[dev], "expr_jit") != hipSuccess) {
                (void)hipGetLastError();
                e.ok = false;
                g_failed.fetch_add(1, std::memory_order_relaxed);
                return declined();
            }
            int nb = 0;
            if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&nb, e.fn[dev], kThreads, 0) != hipSuccess || nb < 1) nb = 2;
            e.per_cu[dev] = nb;
        }
        fn = e.fn[dev];
        per_cu = e.per_cu[dev];
        words = e.words;
    }

    JitArgs g;
    std::memset(&g, 0, sizeof g);
    for (int i = 0; i < n_inputs; ++i) g.in[i] = inputs[i];
    for (int i = 0; i < n_outputs; ++i) g.out[i] = outputs[i];
    g.status = status;
    g.total4 = total / 4;
    g.cols4 = unsigned(cols4);
    g.rows = unsigned(rows);
    g.rows_per_block = 1;
    dim3 grid(1, 1, 1);
    if (!columns) {
        const size_t per_block = size_t(kThreads) * size_t(words);
        const size_t blocks = (g.total4 + per_block - 1) / per_block;
        if (blocks > 0x7fffffffu) return declined();
        grid.x = unsigned(blocks);
    } else {
        const size_t per_block = size_t(kThreads) * size_t(words);
        const size_t gx = (cols4 + per_block - 1) / per_block;
        // enough blocks to fill the chip a few times over, runs of at least 16 rows where the matrix
        // has them: what is computed once per thread is then a small part of its work
        const size_t cus = size_t(compute_units() > 0 ? compute_units() : 256);
        size_t want = cus * size_t(per_cu) * 2;
        size_t gy = (want + gx - 1) / gx;
        if (gy < 1) gy = 1;
        size_t rpb = (rows + gy - 1) / gy;
        if (rpb < 16) rpb = 16;
        if (rpb > rows) rpb = rows;
        gy = (rows + rpb - 1) / rpb;
        if (gx > 0x7fffffffu || gy > 65535) {
            rpb = (rows + 65534) / 65535;
            gy = (rows + rpb - 1) / rpb;
        }
        g.rows_per_block = unsigned(rpb);
        grid.x = unsigned(gx);
        grid.y = unsigned(gy);
    }
    size_t arg_size = sizeof g;
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &g, HIP_LAUNCH_PARAM_BUFFER_SIZE, &arg_size, HIP_LAUNCH_PARAM_END};
    const hipError_t err = hipModuleLaunchKernel(fn, grid.x, grid.y, 1, kThreads, 1, 1, 0, as_stream(stream), nullptr, config);
    if (err != hipSuccess) return fail(CTAMD_EHIP, "ctamd_expr_run_f32: launch of a compiled expression: %s", hipGetErrorString(err));
    g_jit_launches.fetch_add(1, std::memory_order_relaxed);
    return CTAMD_OK;
}

}  // namespace ctamd

using namespace ctamd;

extern "C" int ctamd_set_expr_jit(int threshold) {
    if (threshold < 0) return fail(CTAMD_EINVAL, "%s: negative threshold", __func__);
    g_threshold.store(threshold, std::memory_order_relaxed);
    return CTAMD_OK;
}
extern "C" int ctamd_expr_jit(void) { return g_threshold.load(std::memory_order_relaxed); }
extern "C" void ctamd_expr_jit_stats(uint64_t* compiled, uint64_t* failed, uint64_t* compiled_launches, uint64_t* interpreted_launches) {
    if (compiled) *compiled = g_compiled.load();
    if (failed) *failed = g_failed.load();
    if (compiled_launches) *compiled_launches = g_jit_launches.load();
    if (interpreted_launches) *interpreted_launches = g_interp_launches.load();
}
extern "C" int ctamd_expr_jit_compile(const ctamd_expr_insn* prog, int n_insn, int columns, int words, char* text, size_t cap, size_t* code_bytes) {
    if (!prog || n_insn <= 0 || n_insn > CTAMD_EXPR_MAX_INSNS) return fail(CTAMD_EINVAL, "%s: no program", __func__);
    if (words != 1 && words != 2 && words != 4) return fail(CTAMD_EINVAL, "%s: words per lane must be 1, 2 or 4", __func__);
    for (int pc = 0; pc < n_insn; ++pc)
        if (prog[pc].op > CTAMD_EX_STORE_ZP) return fail(CTAMD_EINVAL, "%s: instruction %d has unknown operator %d", __func__, pc, prog[pc].op);
    const std::string src = generate(prog, n_insn, fast_math(), columns != 0, words);
    if (src.empty()) return fail(CTAMD_EINVAL, "%s: the program reads a slot nobody wrote", __func__);
    if (text && cap) {
        const size_t m = src.size() < cap - 1 ? src.size() : cap - 1;
        std::memcpy(text, src.data(), m);
        text[m] = 0;
    }
    std::vector<char> code;
    std::string log;
    if (!compile(src, code, log)) return fail(CTAMD_EHIP, "%s: %s", __func__, log.c_str());
    if (code_bytes) *code_bytes = code.size();
    return CTAMD_OK;
}
