"""The C-ABI library loads and exports every symbol include/*.h declares (no compute calls: no GPU needed)."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KERNELS = os.path.join(ROOT, "llama.cpp_amd", "lib", "libmi355_kernels.so")
PLUGIN = os.path.join(ROOT, "llama.cpp_amd", "lib", "libggml-mi355.so")


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:mi355|ggml_backend)_[a-z0-9_]+)\s*\(", text)))


def exported(path):
    out = subprocess.run(["nm", "-D", "--defined-only", path], stdout=subprocess.PIPE, text=True, check=True).stdout
    return {l.split()[-1] for l in out.splitlines() if l.strip()}


def test_kernel_library_exports_every_declared_symbol():
    assert os.path.exists(KERNELS), "run build() first"
    names = declared("mi355_kernels.h")
    assert len(names) >= 25
    missing = [n for n in names if n not in exported(KERNELS)]
    assert not missing, missing
    lib = ctypes.CDLL(KERNELS)
    lib.mi355_abi_version.restype = ctypes.c_int
    assert lib.mi355_abi_version() == 1
    lib.mi355_act_bytes.restype = ctypes.c_size_t
    lib.mi355_act_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64]
    assert lib.mi355_act_bytes(4096, 2) == 2 * 4096 + 2 * 128 * 8


def test_python_binding_covers_the_header():
    import mi355
    names = set(declared("mi355_kernels.h"))
    assert names == set(mi355._SIGNATURES), names ^ set(mi355._SIGNATURES)
    mi355.load()


def test_plugin_exports_registry_entry_points():
    if not os.path.exists(PLUGIN):
        pytest.skip("plug-in not built (needs the llama.cpp headers at build time)")
    ex = exported(PLUGIN)
    for n in declared("ggml_mi355.h"):
        assert n in ex, n
    assert {"ggml_backend_init", "ggml_backend_score"} <= ex


def test_argument_errors_are_reported_not_crashed():
    lib = ctypes.CDLL(KERNELS)
    lib.mi355_last_error.restype = ctypes.c_char_p
    lib.mi355_mul_mat_vec_q.restype = ctypes.c_int
    lib.mi355_mul_mat_vec_q.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 3 + [ctypes.c_int64] * 4
    # unsupported type and bad shapes are rejected before any launch
    assert lib.mi355_mul_mat_vec_q(None, 10, None, None, None, 16, 256, 1, 16) == -1   # 10: Q2_K, no kernel here
    assert b"unsupported" in lib.mi355_last_error()
    assert lib.mi355_mul_mat_vec_q(None, 12, None, None, None, 16, 100, 1, 16) == -1
    assert lib.mi355_mul_mat_vec_q(None, 12, None, None, None, 16, 256, 33, 16) == -1
