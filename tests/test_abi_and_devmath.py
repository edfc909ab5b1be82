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
               "ctamd_counters_read"}
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
