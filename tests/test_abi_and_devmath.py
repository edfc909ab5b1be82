"""CPU-side checks of the product's boundary: the shared libraries load, export every entry point
that include/ctorch_amd.h declares (no compute calls without a GPU), the ctypes table matches the
header, and the device math header - compiled unchanged for the host - returns glibc's floats."""
import ctypes as C
import os
import re
import subprocess

import pytest

from support import HOST_LIB, ROOT

HEADER = os.path.join(ROOT, "include", "ctorch_amd.h")


def declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ctamd_\w+)\s*\(", text)))


def test_library_exports_every_declared_entry_point():
    from ctorch_amd import capi
    lib = capi.load()
    names = declared()
    assert len(names) >= 55
    for n in names:
        assert hasattr(lib, n), n
    untyped = {"ctamd_device_count", "ctamd_last_error", "ctamd_version", "ctamd_counters_reset",
               "ctamd_counters_read", "ctamd_expr_jit_stats"}
    assert set(names) - untyped == set(capi.PROTOTYPES), set(names) ^ set(capi.PROTOTYPES)
    assert b"gfx950" in lib.ctamd_version()


def test_no_device_is_an_error_code_not_a_crash():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from ctorch_amd import capi
    lib = capi.load()
    assert lib.ctamd_init(0) == -4 and b"no HIP device" in lib.ctamd_last_error()
    assert lib.ctamd_add_f32(None, None, None, 0, None) == 0              # n == 0 is a no-op
    assert lib.ctamd_add_f32(None, None, None, 4, None) == -1             # null pointers are refused
    assert lib.ctamd_matmul_f32(None, 1, 1, None, 1, 1, None, -1, 1, 1, None) == -1


def test_host_front_end_library_loads_and_exports_its_test_doorway():
    # the doorway is a library of its own; the product library carries none of it
    product = C.CDLL(os.path.join(ROOT, "ctorch_amd", "host", "libctorch_amd_host.so"))
    assert not hasattr(product, "cth_binary") and not hasattr(product, "cth_time_matmul")
    lib = C.CDLL(HOST_LIB)
    for n in ("binary", "unary", "scalar", "sum", "softmax", "matmul_t", "grad_unary", "grad_softmax", "grad_binary",
              "grad_loss", "chain", "mlp_step", "expr", "quiet", "set_reference_row0"):
        assert hasattr(lib, "cth_" + n), n


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from ctorch_amd import capi
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(capi.CtamdError):
        capi.load()


def test_device_math_matches_glibc_on_a_strided_sweep(tmp_path):
    """Every 251st float (17 million inputs, all exponents): expf, sinf, cosf, logf of
    ctorch_amd/csrc/devmath.h against the installed glibc (no mismatch), tanf within 1 ulp, the
    single-precision sine / cosine within 2 ulp.  Run with stride 1 for all 2^32."""
    exe = str(tmp_path / "devmath_check")
    subprocess.check_call(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-mfma", "-o", exe,
                           os.path.join(ROOT, "tests", "native", "devmath_check.c"), "-lm"])
    out = subprocess.check_output([exe, "251"], text=True)
    print(out)
    for line in out.strip().splitlines():
        f = line.split()
        # (the single-precision sine / cosine pair is defined for |x| < 120 only: about half of all floats)
        assert int(f[2]) > (8_000_000 if "_f32" in f[0] else 17_000_000) and int(f[4]) == 0, line


def test_double_exponential_is_glibcs(tmp_path):
    """cta_exp64 (the exponential of the double softmax kernels) against the installed glibc's exp on 16
    million random arguments: the whole range, around zero, the overflow threshold, the subnormal
    results, special values.  No mismatch."""
    exe = str(tmp_path / "exp64_check")
    subprocess.check_call(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-mfma", "-o", exe,
                           os.path.join(ROOT, "tests", "native", "exp64_check.c"), "-lm"])
    out = subprocess.check_output([exe, "2000000"], text=True)
    print(out)
    f = out.split()
    assert f[0] == "tested" and int(f[1]) > 16_000_000 and int(f[3]) == 0, out


def test_division_through_a_double_reciprocal_is_ieee_division(tmp_path):
    """cta_div_rcp (softmax normalisation, x / n in the loss gradients, tensor / scalar) against a / b
    on 64 million random pairs incl. subnormals, and on the 63 million operand pairs whose exact quotient
    is a midpoint between two subnormal floats (where the plain product would break the tie wrongly)."""
    exe = str(tmp_path / "divcheck")
    subprocess.check_call(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-o", exe,
                           os.path.join(ROOT, "tests", "native", "divcheck.c"), "-lm"])
    out = subprocess.check_output([exe, "1000000"], text=True)
    print(out)
    rand, ties = [l.split() for l in out.strip().splitlines()[-2:]]
    assert rand[0] == "tested" and int(rand[1]) == 64_000_000 and int(rand[3]) == 0
    assert ties[0] == "ties" and int(ties[1]) > 60_000_000 and int(ties[3]) == 0


def test_refined_reciprocal_is_correctly_rounded(tmp_path):
    """cta_rcp_refined (the quotient of the single-precision sigmoid): from any starting value within
    1 ulp, two Newton steps give the correctly rounded 1 / s for every significand except all ones,
    where the result is the float below - the case the sigmoid's 2-ulp argument treats separately."""
    exe = str(tmp_path / "rcpcheck")
    subprocess.check_call(["gcc", "-O2", "-ffp-contract=off", "-mfma", "-o", exe,
                           os.path.join(ROOT, "tests", "native", "rcpcheck.c"), "-lm"])
    f = subprocess.check_output([exe], text=True).split()
    assert f[0] == "tested" and int(f[1]) == 3 << 23 and int(f[3]) == 0 and int(f[5]) <= 3, f


def test_fused_expression_kernels_generate_and_compile_without_a_gpu():
    """The run-time compiler path of fused expressions, up to the code object: the kernel text
    generated for the config-5 expression (column-owning pattern, the row vector's reciprocals hoisted)
    and for random programs (both patterns, both math modes) compiles for gfx950."""
    import ctypes as C
    from ctorch_amd import capi
    from support import EX, random_slot_program
    lib = capi.load()

    class Insn(C.Structure):
        _fields_ = [("op", C.c_uint8), ("dst", C.c_uint8), ("a", C.c_uint8), ("b", C.c_uint8), ("imm", C.c_float)]

    def compile_(prog, columns, words):
        arr = (Insn * len(prog))(*[Insn(*q) for q in prog])
        text = C.create_string_buffer(1 << 20)
        size = C.c_size_t(0)
        rc = lib.ctamd_expr_jit_compile(arr, len(prog), columns, words, text, len(text), C.byref(size))
        assert rc == 0, lib.ctamd_last_error().decode()[:4000]
        assert size.value > 1000
        return text.value.decode()

    E = EX
    c5 = [(E["LOAD_FULL"], 0, 0, 0, 0.0), (E["LOAD_ROW"], 1, 1, 0, 0.0), (E["DIV"], 2, 0, 1, 0.0), (E["SIGMOID"], 2, 2, 0, 0.0),
          (E["TANH"], 3, 0, 0, 0.0), (E["SIN"], 4, 0, 0, 0.0), (E["MUL"], 3, 3, 4, 0.0), (E["SUB"], 2, 2, 3, 0.0),
          (E["NEG"], 3, 0, 0, 0.0), (E["COS"], 3, 3, 0, 0.0), (E["ADD"], 2, 2, 3, 0.0), (E["STORE"], 0, 2, 0, 0.0)]
    prev = lib.ctamd_math_mode()
    try:
        for mode in (0, 1):
            assert lib.ctamd_set_math_mode(mode) == 0
            text = compile_(c5, 1, 1)
            assert "1.0 / (double)v1[e]" in text and "cta_div_rcp(v0[e], q1[e])" in text      # the divisor's reciprocal, once per thread
            assert ("sigmoid_fast(v3, tabs)" in text) == (mode == 0)
            compile_(random_slot_program(5, n_full=2, n_row=2, n_ops=24, n_out=3), 1, 2)
            compile_(random_slot_program(6, n_full=3, n_row=0, n_ops=18, n_out=2), 0, 4)
    finally:
        lib.ctamd_set_math_mode(prev)
    bad = (Insn * 1)(Insn(E["ADD"], 0, 1, 2, 0.0))
    assert lib.ctamd_expr_jit_compile(bad, 1, 0, 2, None, 0, None) == -1


def test_no_kernel_spills_registers():
    """The build records what every kernel needs (ctorch_amd/kernel_resources.json, written by
    ctorch_amd.build).  A kernel that spills registers reloads them with waits that also wait for its
    prefetched loads - the one-pass cross entropy lost a quarter of its speed to 25 spilled registers -
    so a build with a spill or a per-lane scratch frame is refused."""
    import json
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ctorch_amd", "kernel_resources.json")
    if not os.path.exists(path):
        pytest.skip("the library was not built by ctorch_amd.build here")
    table = json.load(open(path))
    assert len(table) > 150
    bad = {k: v for k, v in table.items() if v.get("VGPRs Spill", 0) or v.get("ScratchSize [bytes/lane]", 0)}
    assert not bad, bad
