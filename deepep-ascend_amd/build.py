"""Builds, in-tree: libdeep_ep_hip.so (hand-written gfx950 kernels + C ABI) with hipcc, and the `deep_ep._C` extension
(host class `ElasticBuffer` / `EventHandle` over that ABI, csrc/host/) with the host compiler.

Usage: python deepep-ascend_amd/build.py [--software-fp8] [--no-extension]
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "deep_ep")
LIB_NAME = "libdeep_ep_hip.so"
STAMPS_LIB_NAME = "libdeep_ep_hip_stamps.so"     # measurement build: mover wavefronts record their start and end (bench.py --wave-spans)
SOURCES = ["layout.hip", "dispatch.hip", "combine.hip", "low_latency.hip", "api.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def lib_path() -> str:
    return os.path.join(OUT_DIR, LIB_NAME)


def stamps_lib_path() -> str:
    return os.path.join(OUT_DIR, STAMPS_LIB_NAME)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_library(force: bool = True, software_fp8: bool = False, verbose: bool = True) -> str:
    """Compile every kernel source for gfx950 and link the shared library. Returns its path."""
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    flags = list(HIPCC_FLAGS)
    if software_fp8:
        flags.append("-DDEEP_EP_HIP_SOFTWARE_FP8=1")
    hipcc = _hipcc()

    def compile_one(src):
        stamped = src.startswith("stamps:")
        src = src.split(":")[-1]
        obj = os.path.join(obj_dir, src.replace(".hip", "_stamps.o" if stamped else ".o"))
        cmd = [hipcc, *flags, *(["-DDEEP_EP_HIP_WAVE_STAMPS"] if stamped else []), "-c", os.path.join(CSRC, src), "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        # the host pass does not know the packed-fp32 feature and says so; that note is harmless
        err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{res.stderr}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(len(SOURCES) + 1, 8)) as pool:
        objs = list(pool.map(compile_one, SOURCES + ["stamps:dispatch.hip"]))
    stamped_dispatch = objs.pop()
    out = lib_path()
    for target, members in ((out, objs), (stamps_lib_path(), [stamped_dispatch if o.endswith("dispatch.o") else o for o in objs])):
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *members, "-o", target]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stderr}")
        if verbose:
            print(f"built {target}")
    return out


def extension_path() -> str:
    return os.path.join(OUT_DIR, "_C" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_extension(verbose: bool = True) -> str:
    """Compile csrc/host/binding.cpp into deep_ep/_C<ext suffix> and link it against libdeep_ep_hip.so (which must have
    been built).  No device code lives in the extension, so the host compiler does it alone."""
    import pybind11
    import torch
    torch_dir = os.path.dirname(torch.__file__)
    torch_lib = os.path.join(torch_dir, "lib")
    out = extension_path()
    cxx = os.environ.get("CXX", "g++")
    cmd = [
        cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-sign-compare",
        "-DDEEP_EP_PLATFORM_HIP", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        "-I" + os.path.join(torch_dir, "include"), "-I" + os.path.join(torch_dir, "include", "torch", "csrc", "api", "include"),
        "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"], "-I" + pybind11.get_include(),
        os.path.join(CSRC, "host", "binding.cpp"), "-o", out,
        "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
        "-L/opt/rocm/lib", "-lamdhip64", "-L" + OUT_DIR, "-ldeep_ep_hip",
        "-Wl,-rpath," + torch_lib, "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib",
    ]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"building the deep_ep._C extension failed:\n{res.stderr[-4000:]}")
    if verbose:
        if res.stderr.strip():
            print(res.stderr, file=sys.stderr)
        print(f"built {out}")
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--software-fp8", action="store_true", help="use the integer e4m3 encoder instead of v_cvt_pk_fp8_f32")
    ap.add_argument("--no-extension", action="store_true", help="only the kernel library, not the deep_ep._C extension")
    args = ap.parse_args()
    build_library(software_fp8=args.software_fp8)
    if not args.no_extension:
        build_extension()
