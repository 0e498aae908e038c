"""Builds gemm_amd/libqlinear.so from the HIP sources in gemm_amd/csrc for gfx950.

    python -m gemm_amd.build            # compile every translation unit and link

hipcc cross-compiles without a GPU. Packed-FP32 instruction selection is switched off for all
device code (-Xclang -target-feature -Xclang -packed-fp32-ops).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libqlinear.so")
TF_LIB = os.path.join(HERE, "libqlinear_tf.so")
SOURCES = ["qlin_api.hip", "dequant.hip", "gemv_generic.hip", "gemv_q4k.hip", "gemv_stream.hip", "gemv_int.hip", "gemv_grid.hip", "gemm_q4k_mfma.hip", "gemm_kq_wave4.hip", "gemm_kq_wave4s.hip", "gemm_dense_mfma.hip", "moe.hip", "moe_ffn_q4k.hip", "argmax.hip", "gguf_upload.hip", "probe.hip", "gemm_dense_lt.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    cmd = ["hipcc"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    if err:
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lhipblaslt"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB, os.path.getsize(LIB), "bytes")
    build_host(verbose)
    return LIB


def build_host(verbose=True):
    """The plain-C layer with the reference's call shapes (libqlinear_tf.so) and its C test program."""
    inc = os.path.join(os.path.dirname(HERE), "include")
    common = ["gcc", "-O2", "-std=c11", "-Wall", "-Wextra", "-fPIC", "-I", inc]
    link = ["-L", HERE, "-lqlinear", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(common + ["-shared", "-o", TF_LIB, os.path.join(HERE, "host", "qlinear_tf.c")] + link,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("gcc failed on qlinear_tf.c:\n" + r.stderr)
    tests_c = os.path.join(os.path.dirname(HERE), "tests", "c")
    exe = os.path.join(tests_c, "test_tf_mirror")
    r = subprocess.run(common + ["-o", exe, os.path.join(tests_c, "test_tf_mirror.c"), "-L", HERE, "-lqlinear_tf",
                                 "-lqlinear", "-lm", "-Wl,-rpath,$ORIGIN/../../gemm_amd"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("gcc failed on test_tf_mirror.c:\n" + r.stderr)
    if r.stderr.strip():
        sys.stderr.write(r.stderr)
    if verbose:
        print("built", TF_LIB, "and", exe)


if __name__ == "__main__":
    build()
