"""Builds lbann_amd/liblbnorm.so: the HIP kernels and their C ABI, for gfx950 only.

    python -m lbann_amd.build

hipcc cross-compiles without a GPU.  The library depends on the HIP runtime only
(no torch, no MPI).  Packed-fp32 VALU instructions are switched off for every
translation unit.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblbnorm.so")
SOURCES = ["capi_common.hip", "softmax.hip", "layer_norm.hip", "batch_norm.hip", "entrywise_batch_norm.hip",
           "entrywise_batch_norm_split.hip", "cross_entropy.hip", "scale_bias.hip", "gradient_sink.hip", "f64_layers.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src, extra=(), tag=""):
    obj = os.path.join(CSRC, src.replace(".hip", tag + ".o"))
    subprocess.run([HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj], check=True)
    return obj


def build(jobs: int = 4, extra=(), lib: str = LIB, tag: str = "") -> str:
    """`extra` adds compiler flags (e.g. -DLBN_NT_STORE=0) and `lib`/`tag` name an alternative
    output, for side-by-side experiments; lbann_amd.capi loads $LBN_LIB when it is set."""
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra, tag), SOURCES))
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs], check=True)
    return lib


def build_adapter_driver() -> str:
    """Compiles tests/cpp/adapter_driver.cpp (host code over the header-only C++ adapter)
    into tests/cpp/libadapter_driver.so, linked against liblbnorm.so."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "cpp", "adapter_driver.cpp")
    out = os.path.join(root, "tests", "cpp", "libadapter_driver.so")
    subprocess.run([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared",
                    "-Wall", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", src, "-o", out,
                    "-L" + HERE, "-llbnorm", "-Wl,-rpath,$ORIGIN/../../lbann_amd"], check=True)
    return out


if __name__ == "__main__":
    print(build())
    print(build_adapter_driver())
    sys.exit(0)
