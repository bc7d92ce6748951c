"""Build recipe for libhipattn.so (HIP kernels + C ABI), gfx950 only.

hipcc cross-compiles without a GPU.  The library is built in-tree, next to the sources
(openvino_contrib_amd/csrc/libhipattn.so), so that it travels with the source tree.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(_HERE), "include")
LIB_PATH = os.path.join(CSRC, "libhipattn.so")

SOURCES = [
    "hipattn_api.hip",
    "kv_cache_write.hip",
    "attention_generic.hip",
    "paged_decode.hip",
    "paged_scores.hip",
    "flash_prefill.hip",
    "flash_small.hip",
]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # keep hipcc from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + INCLUDE,
    "-I" + CSRC,
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libhipattn cannot be built")
    return exe


def _compile(src, extra):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc()] + HIPCC_FLAGS + list(extra) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, r.stderr[-4000:]))
    return obj, r.stderr


def _build_shared(sources, lib_path, verbose, extra_flags, jobs, link_flags=()):
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda s: _compile(s, extra_flags), sources))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            lines = [l for l in err.splitlines() if "packed-fp32-ops" not in l]
            if lines:
                print("\n".join(lines), file=sys.stderr)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path] + objs + list(link_flags)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr[-4000:])
    for o in objs:
        os.remove(o)
    return lib_path


def build_library(verbose=False, extra_flags=(), jobs=4):
    """Compile every HIP source and link libhipattn.so.  Always recompiles."""
    return _build_shared(SOURCES, LIB_PATH, verbose, extra_flags, jobs)


OPS_LIB_PATH = os.path.join(CSRC, "libhipops.so")
OPS_SOURCES = ["ops/hipops_api.hip", "ops/layer_ops.hip", "ops/format_ops.hip", "ops/math_ops.hip", "ops/matmul.hip"]


def build_ops_library(verbose=False, extra_flags=(), jobs=4):
    """libhipops.so: the operators around attention (RMS norm, RoPE, MatMul over hipBLASLt, Gather,
    Concat, the gated MLP's element-wise operators, Transpose, Convert).  A library of its own because it links hipBLASLt."""
    return _build_shared(OPS_SOURCES, OPS_LIB_PATH, verbose, extra_flags, jobs, link_flags=["-lhipblaslt"])


YARDSTICK_LIB_PATH = os.path.join(CSRC, "bench", "libmfma_yardstick.so")


def build_bench_tools():
    """The yardsticks of bench.py --workload mfma and --workload stream: a library of its own, not part of libhipattn."""
    sources = [os.path.join(CSRC, "bench", name) for name in ("mfma_yardstick.hip", "stream_yardstick.hip")]
    cmd = [hipcc()] + HIPCC_FLAGS + ["-shared"] + sources + ["-o", YARDSTICK_LIB_PATH]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on the yardsticks:\n%s" % r.stderr[-4000:])
    return YARDSTICK_LIB_PATH


PLUGIN_LIB_PATH = os.path.join(CSRC, "libhip_plugin.so")
PLUGIN_SOURCES = ["plugin/src/hip_ops.cpp", "plugin/src/hip_layer_ops.cpp", "plugin/src/hip_format_ops.cpp", "plugin/src/hip_math_ops.cpp", "plugin/src/hip_plugin.cpp", "plugin/src/hip_create_plugin.cpp",
                  "plugin/test_facade/c_api.cpp"]


def build_plugin():
    """Compile the host-side plugin layer (plain C++17, reaches the GPU only through libhipattn's C ABI)
    against the stand-in for OpenVINO's developer headers (plugin/standin/), plus the C facade the
    tests drive it through.  Where the OpenVINO developer package is installed, plugin/CMakeLists.txt
    builds the same sources against the real headers instead."""
    if not os.path.exists(LIB_PATH) or not os.path.exists(OPS_LIB_PATH):
        raise RuntimeError("build libhipattn.so and libhipops.so first")
    cxx = shutil.which("g++") or "g++"
    cmd = [cxx, "-std=c++17", "-O2", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-Wextra", "-pthread",
           "-I" + INCLUDE, "-I" + os.path.join(CSRC, "plugin", "src"), "-I" + os.path.join(CSRC, "plugin", "standin")]
    cmd += [os.path.join(CSRC, s) for s in PLUGIN_SOURCES]
    cmd += ["-L" + CSRC, "-lhipattn", "-lhipops", "-Wl,-rpath,$ORIGIN", "-o", PLUGIN_LIB_PATH]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("plugin build failed:\n%s" % r.stderr[-6000:])
    return PLUGIN_LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_ops_library(verbose=True))
    print(build_plugin())
    print(build_bench_tools())
