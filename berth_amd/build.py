"""Compile the HIP sources under berth_amd/csrc for gfx950 into in-tree shared
libraries (berth_amd/lib/*.so).  hipcc cross-compiles without a GPU."""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "lib", "obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU ops are switched off for every device compilation
# no implicit mul+add fusion: the Hadamard butterflies must round like the CPU oracle
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-result", "-Wno-unknown-warning-option"]

LIBRARIES = {
    "libberth_kernels_hip.so": ["api.hip", "exl3_gemv.hip", "exl3_gemv_cb0.hip", "exl3_gemv_cb1.hip",
                                "exl3_gemv_cb2.hip", "exl3_gemv_stream_cb0.hip", "exl3_gemv_stream_cb1.hip",
                                "exl3_gemv_stream_cb2.hip", "exl3_gemm.hip", "exl3_gemm_cb0.hip", "exl3_gemm_cb1.hip",
                                "exl3_gemm_cb2.hip",
                                "exl3_reconstruct.hip", "elementwise.hip", "moe.hip"],
    "libberth_hip.so": ["berth_hip.hip"],
}


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0].replace("/", "_") + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
    return obj


def build_all(jobs: int = 8, only: str | None = None) -> list[str]:
    os.makedirs(OBJ, exist_ok=True)
    libs = {k: v for k, v in LIBRARIES.items() if only in (None, k)}
    sources = sorted({s for v in libs.values() for s in v if os.path.exists(os.path.join(CSRC, s))})
    with cf.ThreadPoolExecutor(max_workers=min(jobs, 16)) as ex:
        objs = dict(zip(sources, ex.map(_compile, sources)))
    built = []
    for name, srcs in libs.items():
        have = [objs[s] for s in srcs if s in objs]
        if not have:
            continue
        out = os.path.join(LIB, name)
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *have, "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed for {name}:\n{r.stderr[-4000:]}")
        built.append(out)
    if only is None:
        built.append(build_code_object())
        built.append(build_reader())
        built.append(build_host_check())
        built.append(build_bench_native())
    return built


def build_bench_native() -> str:
    """bench.py's native helpers (bench_native.hip at the repository root: the vector-ALU rate
    probe and the eager launch loop over the C ABI), linked against the kernels library."""
    root = os.path.dirname(HERE)
    out = os.path.join(root, "libberth_bench.so")
    cmd = [HIPCC, *FLAGS, "-shared", "-I" + root, os.path.join(root, "bench_native.hip"), "-o", out,
           "-L" + LIB, "-lberth_kernels_hip", "-Wl,-rpath,$ORIGIN/berth_amd/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"bench helper build failed:\n{r.stderr[-4000:]}")
    return out


def build_code_object() -> str:
    """A stand-alone gfx950 code object (hipcc --genco) with the test kernels the runtime
    library's module path is exercised with (tests/runtime_probe.hip, tests/test_gpu_runtime.py)."""
    tests = os.path.join(os.path.dirname(HERE), "tests")
    out = os.path.join(tests, "runtime_probe.hsaco")
    cmd = [HIPCC, "--genco", "--offload-arch=gfx950", "-O3", "-ffp-contract=off",
           os.path.join(tests, "runtime_probe.hip"), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"code object build failed:\n{r.stderr[-4000:]}")
    return out


def build_reader() -> str:
    """The EXL3 checkpoint reader and the model planner (csrc/host/exl3_reader_capi.cpp,
    plan_capi.cpp): host-only C++ in one library."""
    out = os.path.join(LIB, "libberth_exl3_reader.so")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-Wall",
           os.path.join(CSRC, "host", "exl3_reader_capi.cpp"), os.path.join(CSRC, "host", "plan_capi.cpp"), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"checkpoint reader build failed:\n{r.stderr[-4000:]}")
    return out


def build_host_check() -> str:
    """The C++ host layer's check program (csrc/host): plain C++ over the two C ABIs."""
    out = os.path.join(LIB, "berth_host_check")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", os.path.join(CSRC, "host", "host_check.cpp"), "-o", out,
           "-L" + LIB, "-lberth_kernels_hip", "-lberth_hip", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"host check build failed:\n{r.stderr[-4000:]}")
    return out


if __name__ == "__main__":
    for path in build_all(only=sys.argv[1] if len(sys.argv) > 1 else None):
        print("built", path)
