"""Build recipe of the native parts.

  kernels : llama.cpp_amd/lib/libmi355_kernels.so  - HIP kernels + C ABI (include/mi355_kernels.h)
  backend : llama.cpp_amd/lib/libggml-mi355.so     - the ggml backend plug-in; compiled against
            the llama.cpp headers, so it is only (re)built where a llama.cpp tree is present
            (LLAMA_CPP_DIR, default /root/reference).

Both are built for gfx950 only, in-tree, with hipcc.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))       # llama.cpp_amd/
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
BACKEND_SRC = os.path.join(PKG, "backend")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(LIB, "obj")

KERNEL_SOURCES = ["quantize.hip", "wquant.hip", "gemv.hip", "ffn.hip", "mul_mat.hip", "skinny.hip", "mid.hip", "mmq.hip", "mmq_k.hip", "mmq_w.hip", "mul_mat_id.hip", "fattn.hip", "fattn_mma.hip", "fattn_stream.hip", "kv_quant.hip", "glue.hip", "fused.hip", "moe.hip"]

# -packed-fp32-ops: keep hipcc from forming packed-FP32 instructions out of scalar float code
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        sys.stderr.write(out + "\n")
        raise RuntimeError("command failed: " + " ".join(cmd))
    return out


def kernels_lib_path():
    return os.path.join(LIB, "libmi355_kernels.so")


def backend_lib_path():
    return os.path.join(LIB, "libggml-mi355.so")


def build_kernels(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    objs = []

    def compile_one(src):
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        _run([_hipcc()] + HIPCC_FLAGS + ["-I", os.path.join(ROOT, "include"), "-c", os.path.join(CSRC, src), "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(KERNEL_SOURCES))) as ex:
        objs = list(ex.map(compile_one, KERNEL_SOURCES))
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", kernels_lib_path()] + objs)
    if verbose:
        print("built", kernels_lib_path())
    return kernels_lib_path()


def build_backend(llama_dir=None, verbose=True):
    llama_dir = llama_dir or os.environ.get("LLAMA_CPP_DIR", "/root/reference")
    hdr = os.path.join(llama_dir, "ggml", "src", "ggml-backend-impl.h")
    if not os.path.exists(hdr):
        if verbose:
            print("no llama.cpp tree at %s: keeping the prebuilt %s" % (llama_dir, backend_lib_path()))
        return None
    src = os.path.join(BACKEND_SRC, "ggml_mi355.cpp")
    if not os.path.exists(src):
        return None
    os.makedirs(LIB, exist_ok=True)
    _run([_hipcc()] + HIPCC_FLAGS + ["-x", "hip", "-DGGML_BACKEND_DL", "-DGGML_BACKEND_SHARED", "-DGGML_BACKEND_BUILD",
                                     "-I", os.path.join(ROOT, "include"),
                                     "-I", os.path.join(llama_dir, "ggml", "include"), "-I", os.path.join(llama_dir, "ggml", "src"),
                                     "-shared", src, "-o", backend_lib_path(),
                                     "-L", LIB, "-lmi355_kernels", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built", backend_lib_path())
    return backend_lib_path()


def build_all(verbose=True):
    build_kernels(verbose)
    build_backend(verbose=verbose)


if __name__ == "__main__":
    build_all()
