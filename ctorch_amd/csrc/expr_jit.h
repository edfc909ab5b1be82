// Run-time compiled kernels for fused elementwise expressions (expr_jit.hip), as the launcher of
// expr.hip sees them.
#ifndef CTAMD_EXPR_JIT_H
#define CTAMD_EXPR_JIT_H

#include "common.h"

namespace ctamd {

constexpr int kJitDeclined = 1;   // not launched: the interpreter takes the program

// Launches the compiled kernel for `prog` (already validated; aligned: every pointer 16-byte aligned,
// total and cols multiples of four, fewer than 2^32 words - anything else is declined) when there is one, compiling it first when the
// program has now been seen often enough.  Returns CTAMD_OK when it launched, kJitDeclined when
// the interpreter has to run the program, a negative code when the launch itself failed.
int jit_try_launch(const ctamd_expr_insn* prog, int n_insn, const float* const* inputs, int n_inputs, float* const* outputs, int n_outputs,
                   int32_t* status, size_t rows, size_t cols, bool aligned, bool fastm, void* stream);

}  // namespace ctamd

#endif
