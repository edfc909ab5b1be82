"""ctypes binding of the C ABI in include/ctorch_amd.h (ctorch_amd/libctorch_amd.so).

The library is the product; this module only loads it and declares the prototypes.  There is no
fallback: if the shared library is missing, loading raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libctorch_amd.so")

_P = C.c_void_p
_Z = C.c_size_t
_I64 = C.c_int64

# name -> argument types (all return int)
PROTOTYPES = {
    "ctamd_init": [C.c_int],
    "ctamd_malloc": [C.POINTER(_P), _Z],
    "ctamd_free": [_P],
    "ctamd_memcpy_h2d": [_P, _P, _Z, _P],
    "ctamd_memcpy_d2h": [_P, _P, _Z, _P],
    "ctamd_read_small": [_P, _P, _Z, _P],
    "ctamd_memcpy_d2d": [_P, _P, _Z, _P],
    "ctamd_sync": [_P],
    "ctamd_set_math_mode": [C.c_int],
    "ctamd_math_mode": [],
    "ctamd_stream_create": [C.POINTER(_P)],
    "ctamd_stream_destroy": [_P],
    "ctamd_graph_begin": [_P],
    "ctamd_graph_end": [_P, C.POINTER(_P)],
    "ctamd_graph_launch": [_P, _P],
    "ctamd_graph_destroy": [_P],
}
PROTOTYPES.update({
    "ctamd_div_backward_b_rowbcast_f32": [_P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_u8_to_unit_f32": [_P, _P, _Z, _P],
    "ctamd_onehot_f32": [_P, _P, _Z, _Z, _P],
    "ctamd_sgd_step_f32": [_P, _P, C.c_float, _Z, _P],
    "ctamd_count_correct_f32": [_P, _P, _P, _Z, _Z, _P],
})
for _op in ("add", "sub", "mul", "div"):
    PROTOTYPES["ctamd_%s_f32" % _op] = [_P, _P, _P, _Z, _P]
    PROTOTYPES["ctamd_%s_rowbcast_f32" % _op] = [_P, _P, _P, _Z, _Z, _P]
    PROTOTYPES["ctamd_%s_bscalar_f32" % _op] = [_P, _P, _P, _Z, _P]
PROTOTYPES["ctamd_rsub_ascalar_f32"] = [_P, _P, _P, _Z, _P]
for _op in ("add", "mul", "div"):
    PROTOTYPES["ctamd_%s_scalar_f32" % _op] = [_P, C.c_float, _P, _Z, _P]
for _op in ("neg", "relu", "sin", "cos", "tanh", "sigmoid"):
    PROTOTYPES["ctamd_%s_f32" % _op] = [_P, _P, _Z, _P]
PROTOTYPES.update({
    "ctamd_sum_f32": [_P, _P, _Z, _P],
    "ctamd_dot_f32": [_P, _P, _P, _Z, _P],
    "ctamd_dot_static_f32": [_P, _P, _P, _Z, _P],
    "ctamd_mse_f32": [_P, _P, _P, _Z, _P],
    "ctamd_mae_f32": [_P, _P, _P, _Z, _P],
    "ctamd_colsum_f32": [_P, _P, _Z, _Z, _P],
    "ctamd_any_abs_lt_eps_f32": [_P, _P, _Z, _P],
    "ctamd_softmax_rows_f32": [_P, _P, _Z, _Z, _P],
    "ctamd_softmax_cols_f32": [_P, _P, _Z, _Z, _P],
    "ctamd_cross_entropy_onehot_f32": [_P, _P, _P, _Z, _Z, _P],
    "ctamd_cross_entropy_index_f32": [_P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_cross_entropy_index_stats_f32": [_P, _P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_cross_entropy_backward_index_stats_f32": [_P, _P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_matmul_f32": [_P, _I64, _I64, _P, _I64, _I64, _P, _I64, _I64, _I64, _P],
    "ctamd_sgd_step_multi_f32": [_P, _P, _P, C.c_int, C.c_float, _P],
    "ctamd_compare_f32": [C.c_int, _P, _P, _P, _Z, _P],
    "ctamd_compare_scalar_f32": [C.c_int, _P, C.c_float, _P, _Z, _P],
    "ctamd_cross_entropy_index_fused_f32": [_P, _P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_fill_typed": [_P, C.c_int, C.c_double, _Z, _P],
    "ctamd_cast_from_f32": [_P, _P, C.c_int, _Z, _P],
    "ctamd_scalar_op_typed": [_P, _P, C.c_int, C.c_int, C.c_float, _Z, _P],
    "ctamd_accumulate_typed": [_P, _P, C.c_int, _Z, _P],
    "ctamd_softmax_f64": [_P, _P, _Z, _Z, C.c_int, _P],
    "ctamd_expr_run_f32": [_P, C.c_int, _P, C.c_int, _P, C.c_int, _P, _Z, _Z, _P],
    "ctamd_linear_ce_head_fits": [_Z, _Z],
    "ctamd_linear_ce_head_f32": [_P, _P, _P, _P, _P, _P, _P, _P, _P, C.c_int, _P, _P, _Z, _Z, _Z, _P],
    "ctamd_set_expr_jit": [C.c_int],
    "ctamd_expr_jit": [],
    "ctamd_expr_jit_compile": [_P, C.c_int, C.c_int, C.c_int, _P, _Z, _P],
    "ctamd_matmul_bias_f32": [_P, _I64, _I64, _P, _I64, _I64, _P, C.c_int, _P, _I64, _I64, _I64, _P],
    "ctamd_matmul_relu_mask_f32": [_P, _I64, _I64, _P, _I64, _I64, _P, _P, _I64, _I64, _I64, _P],
    "ctamd_matmul_colsum_f32": [_P, _I64, _I64, _P, _I64, _I64, _P, _P, _I64, _I64, _I64, _P],
    "ctamd_fill_f32": [_P, C.c_float, _Z, _P],
    "ctamd_fill_from_f32": [_P, _P, _Z, _P],
    "ctamd_accumulate_f32": [_P, _P, _Z, _P],
    "ctamd_mse_backward_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_relu_backward_acc_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_sigmoid_backward_acc_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_tanh_backward_acc_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_sin_backward_acc_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_cos_backward_acc_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_mul_acc_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_div_acc_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_div_rowbcast_acc_f32": [_P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_mse_backward_acc_f32": [_P, _P, _P, _P, _P, _Z, _P],
    "ctamd_mae_backward_acc_f32": [_P, _P, _P, _P, _P, _Z, _P],
    "ctamd_mae_backward_f32": [_P, _P, _P, _P, _Z, _P],
    "ctamd_softmax_backward_rows_f32": [_P, _P, _P, _Z, _Z, _P],
    "ctamd_softmax_backward_cols_f32": [_P, _P, _P, _Z, _Z, _P],
    "ctamd_cross_entropy_backward_onehot_f32": [_P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_cross_entropy_backward_index_f32": [_P, _P, _P, _P, _Z, _Z, _P],
    "ctamd_div_backward_b_f32": [_P, _P, _P, _P, _Z, _P],
})
for _op in ("relu", "sigmoid", "tanh", "sin", "cos", "abs", "sqrt", "square", "tan"):
    PROTOTYPES["ctamd_%s_backward_f32" % _op] = [_P, _P, _P, _Z, _P]
for _op in ("abs", "exp", "log", "sqrt", "square", "tan"):
    PROTOTYPES["ctamd_%s_f32" % _op] = [_P, _P, _Z, _P]
PROTOTYPES.update({
    "ctamd_sub_scalar_f32": [_P, C.c_float, _P, _Z, _P],
    "ctamd_leaky_relu_f32": [_P, C.c_float, _P, _Z, _P],
    "ctamd_leaky_relu_backward_f32": [_P, _P, C.c_float, _P, _Z, _P],
    "ctamd_reduce_dim_f32": [C.c_int, _P, _P, _P, _P, _Z, _Z, _Z, C.c_int, _P],
    "ctamd_reduce_dim_backward_f32": [C.c_int, _P, _P, _P, _P, _P, _P, _Z, _Z, _Z, C.c_int, _P],
    "ctamd_fold_mod_f32": [_P, _P, _Z, _Z, _P],
    "ctamd_broadcast_reduce_f32": [_P, _P, _P, C.c_int, _P, _P],
    "ctamd_log_softmax_rows_f32": [_P, _P, _Z, _Z, _P],
    "ctamd_log_softmax_cols_f32": [_P, _P, _Z, _Z, _P],
    "ctamd_log_softmax_backward_rows_f32": [_P, _P, _P, _Z, _Z, _P],
    "ctamd_log_softmax_backward_cols_f32": [_P, _P, _P, _Z, _Z, _P],
})

_lib = None


class CtamdError(RuntimeError):
    pass


def load():
    """Loads libctorch_amd.so (once) and returns the ctypes handle with prototypes set."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CtamdError("%s is missing: build it with `python -m ctorch_amd.build` "
                         "(there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, args in PROTOTYPES.items():
        fn = getattr(lib, name)       # raises AttributeError if the export is missing
        fn.argtypes = args
        fn.restype = C.c_int
    lib.ctamd_device_count.restype = C.c_int
    lib.ctamd_counters_reset.argtypes = []
    lib.ctamd_counters_reset.restype = None
    lib.ctamd_counters_read.argtypes = [C.POINTER(C.c_double)] * 3 + [C.POINTER(C.c_uint64)]
    lib.ctamd_counters_read.restype = None
    lib.ctamd_expr_jit_stats.argtypes = [C.POINTER(C.c_uint64)] * 4
    lib.ctamd_expr_jit_stats.restype = None
    lib.ctamd_last_error.restype = C.c_char_p
    lib.ctamd_version.restype = C.c_char_p
    _lib = lib
    return lib


def counters(lib=None):
    """(algorithmic bytes, flops, seconds at the MI355X peaks, operator launches) since the last
    ctamd_counters_reset()."""
    lib = lib or load()
    b, f, t, n = C.c_double(), C.c_double(), C.c_double(), C.c_uint64()
    lib.ctamd_counters_read(C.byref(b), C.byref(f), C.byref(t), C.byref(n))
    return b.value, f.value, t.value, n.value


def check(rc):
    if rc != 0:
        raise CtamdError("ctorch_amd error %d: %s" % (rc, load().ctamd_last_error().decode()))
