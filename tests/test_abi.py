"""C ABI checks that need no GPU: every function declared in include/faith_amd.h is exported by
the built library, the Python binding lists the same set, and argument validation returns
status codes (nothing is launched, nothing aborts)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "faith_amd.h")


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(faith_\w+)\s*\(", src)))


@pytest.fixture(scope="module")
def lib():
    from faith_amd import _lib
    return _lib


def test_header_declares_the_reference_surface():
    names = declared_functions()
    for fn in ("faith_relu_verification", "faith_tanh_verification", "faith_matmul_verification",
               "faith_dot_product_verification_QK", "faith_convolution_verification", "faith_concretize"):
        assert fn in names


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(lib.LIB_PATH)
    for fn in declared_functions():
        assert hasattr(raw, fn), f"{fn} is declared in include/faith_amd.h but not exported"


def test_binding_covers_every_entry_point(lib):
    bound = set(lib.SIGNATURES) | {"faith_last_error", "faith_version", "faith_static_scratch_bytes"}
    assert set(declared_functions()) == bound


def test_null_and_shape_errors_are_status_codes(lib):
    L = lib.lib
    buf = (ctypes.c_float * 64)()
    p = ctypes.cast(buf, ctypes.c_void_p)          # non-NULL host address; validation fails before any use
    # NULL required pointer
    assert L.faith_concretize(None, p, p, p, p, p, 1, 4, 4, 0.1, lib.Q_2, 1, 0, None) == -1
    assert b"NULL" in L.faith_last_error()
    # non-positive dimension
    assert L.faith_concretize(p, p, p, p, p, p, 0, 4, 4, 0.1, lib.Q_2, 1, 0, None) == -2
    # words must divide dim_in
    assert L.faith_relu_verification(p, p, p, p, p, p, p, p, None, None, 1, 6, 4, 0.1, lib.Q_2, 4, 0, None) == -2
    # unknown norm / layout
    assert L.faith_tanh_verification(p, p, p, p, p, p, p, p, None, None, 1, 4, 4, 0.1, 7, 1, 0, None) == -3
    assert L.faith_tanh_verification(p, p, p, p, p, p, p, p, None, None, 1, 4, 4, 0.1, lib.Q_1, 1, 9, None) == -3
    # misaligned pointer
    q = ctypes.c_void_p(p.value + 2)
    assert L.faith_matmul_verification(q, p, p, p, p, None, p, p, p, p, 1, 1, 4, 4, 4, None) == -4
    assert L.faith_matmul_verification(p, p, p, p, p, None, p, p, p, p, 1, 0, 4, 4, 4, None) == -2
    assert L.faith_dot_product_verification_QK(p, p, p, p, p, p, p, p, p, p, p, p, p, p, p, p,
                                               1, 0, 4, 4, 4, 0.1, lib.Q_1, 1, 0, None) == -2
    assert L.faith_dot_product_verification_QK(p, p, p, p, p, p, p, p, p, p, p, p, p, p, p, p,
                                               1, 0, 4, 4, 4, 0.1, lib.Q_1, 1, 1, None) == -2      # transposed layout
    assert L.faith_dot_product_verification_V(p, p, p, p, p, p, p, p, p, p, p, p, p, p, p, p,
                                              1, 4, 4, 4, 4, 0.1, lib.Q_1, 1, 5, None) == -3       # unknown layout
    # kernel larger than the padded image
    assert L.faith_convolution_verification(p, p, p, p, p, None, p, p, p, p, 1, 2, 2, 1, 1, 5, 1, 0, 1, None) == -2
    assert L.faith_tune_set(99, 1) == -3
    # the driver's launches
    assert L.faith_input_coefficients(None, p, None, 1.0, 1, 4, 1, 8, 0, None) == -1
    assert L.faith_input_coefficients(p, None, None, 1.0, 1, 4, 1, 8, 0, None) == -1     # a dense object needs positions
    assert L.faith_input_coefficients(p, None, None, 1.0, 1, 4, 1, 8, 1, None) == -2     # compact: one row per word
    assert L.faith_flag_below(p, p, 0, 4, 0.0, 1, None) == -2
    assert L.faith_verdict(p, p, None, None, 1, 1, 0, None) == -1
    assert L.faith_concretize_rows(p, p, p, p, None, p, p, 1, 4, 1, 8, 8, 0.1, lib.Q_2, 1, None) == -1
    assert L.faith_concretize_rows(p, p, p, p, p, p, p, 1, 4, 1, 8, 8, 0.1, lib.Q_2, 3, None) == -2   # words divide dim_in
    assert L.faith_concretize_rows(p, p, p, p, p, p, p, 1, 4, 1, 8, 8, 0.1, 7, 1, None) == -3
    # the allocation-free dot product refuses what its 4 MiB array cannot hold, before touching the GPU
    assert L.faith_static_scratch_bytes() == 4 << 20
    assert L.faith_dot_product_verification_QK_static(p, p, p, p, p, p, p, p, p, p, p, p,
                                                      16, 512, 512, 64, 8, 0.1, lib.Q_1, 1, 0, None) == -3
    assert b"scratch" in L.faith_last_error()
    assert L.faith_dot_product_verification_QK_static(p, p, p, p, p, p, p, p, p, p, p, p,
                                                      1, 0, 4, 4, 4, 0.1, lib.Q_1, 1, 0, None) == -2


def test_tuning_knobs_are_kept_per_thread():
    """Concurrent setters never fail, and what a thread that has ended did -- its knob values, the message of its
    refused call -- is not the main thread's (tests/test_gpu_act.py checks on the GPU that a knob set in one thread
    selects that thread's kernels only)."""
    import threading
    from faith_amd import _lib as lib
    L = lib.lib
    codes = []

    def worker(i):
        for _ in range(200):
            codes.append(L.faith_tune_set(i % 5, i))
        codes.append(L.faith_tune_set(99, 1))          # the unknown knob's message stays in this thread

    L.faith_tune_set(0, 0)
    before = L.faith_last_error()
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert codes.count(0) == 8 * 200 and codes.count(-3) == 8
    assert L.faith_last_error() == before


def test_python_wrappers_refuse_cpu_tensors():
    import torch
    from faith_amd import ops
    lw = torch.zeros(1, 2, 4, 4)
    lb = torch.zeros(1, 2, 4)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.relu(lw, lb, lw, lb, 2.0, 0.1)
    with pytest.raises(ValueError):
        ops.q_code(0.5)
    assert ops.q_code(float("inf")) == ops.Q_1 and ops.q_code(1) == ops.Q_INF and ops.q_code(2) == ops.Q_2
    assert ops.q_code(12) == ops.Q_1                       # the reference treats p >= 10 as infinity
    # any other norm: the int carries the bits of the dual exponent (p = 3 -> q = 1.5)
    import struct
    assert struct.unpack("f", struct.pack("i", ops.q_code(3.0)))[0] == 1.5


def test_workloads_are_reproducible():
    import torch
    from faith_amd.workloads import make_config
    a, b = make_config(0), make_config(0)
    assert torch.equal(a["x"]["lw"], b["x"]["lw"]) and torch.equal(a["W"], b["W"])
    assert bool((a["x"]["uw"] >= a["x"]["lw"]).all()) and bool((a["x"]["ub"] >= a["x"]["lb"]).all())
    c3 = make_config(3, scale=0.1)
    assert c3["x"]["lw"].shape == (4, 13, 256, 64)


def test_binding_argument_types_match_the_header(lib):
    """Every prototype in include/faith_amd.h, parameter by parameter, against the ctypes table."""
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    protos = re.findall(r"\bint\s+(faith_\w+)\s*\(([^;]*?)\)\s*;", src, flags=re.S)
    assert len(protos) >= 15
    kinds = {ctypes.c_void_p: "pointer", ctypes.c_int: "int", ctypes.c_float: "float", ctypes.c_longlong: "long long"}
    for name, params in protos:
        if name in ("faith_version",):
            continue
        want = []
        for prm in [x.strip() for x in params.replace("\n", " ").split(",")]:
            if prm in ("void", ""):
                continue
            if "*" in prm:
                want.append("pointer")
            elif prm.startswith("long long"):
                want.append("long long")
            elif prm.startswith("float"):
                want.append("float")
            elif prm.startswith("int"):
                want.append("int")
            else:
                raise AssertionError(f"{name}: cannot classify parameter {prm!r}")
        got = [kinds[t] for t in lib.SIGNATURES[name]]
        assert got == want, f"{name}: header {want} vs binding {got}"


def test_header_and_library_serve_a_plain_c_caller(tmp_path, lib):
    """The boundary is a C ABI: a C99 program that includes the header and links the library calls it
    (version, argument validation -- nothing is launched, so no GPU is needed)."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "caller.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "faith_amd.h"\n'
        "int main(void) {\n"
        "    float buf[16];\n"
        "    if (faith_version() <= 0) return 1;\n"
        "    if (faith_concretize(NULL, buf, buf, buf, buf, buf, 1, 4, 4, 0.1f, FAITH_Q_2, 1, FAITH_LAYOUT_NATURAL, NULL) != FAITH_ERR_NULL) return 2;\n"
        "    if (strstr(faith_last_error(), \"NULL\") == NULL) return 3;\n"
        "    if (faith_concretize(buf, buf, buf, buf, buf, buf, 0, 4, 4, 0.1f, FAITH_Q_2, 1, FAITH_LAYOUT_NATURAL, NULL) != FAITH_ERR_SHAPE) return 4;\n"
        "    if (faith_softmax_fits(256, 32) != 1 || faith_softmax_fits(64, 300) != 0) return 5;\n"
        '    printf("ok %d\\n", faith_version());\n'
        "    return 0;\n}\n")
    exe = tmp_path / "caller"
    libdir = os.path.dirname(lib.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", f"-I{os.path.join(ROOT, 'include')}", str(src),
                    f"-L{libdir}", "-lfaith_amd", f"-Wl,-rpath,{libdir}", "-o", str(exe)], check=True, capture_output=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.startswith("ok"), (out.returncode, out.stdout, out.stderr)
