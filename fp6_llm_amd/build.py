"""Builds fp6_llm_amd/libfp6mi.so (host code + gfx950 kernels + C ABI) with hipcc. Run: python -m fp6_llm_amd.build"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
# (source, object name, extra flags): the kernel file is compiled once per weight format (tag = 10*E + M), the objects in parallel
FORMAT_TAGS = (32, 22, 23, 21)
UNITS = [("fp6mi_host.cpp", "fp6mi_host.o", []), ("fp6mi_api.hip", "fp6mi_api.o", [])] + \
        [("fp6mi_gemm.hip", "fp6mi_gemm_%d.o" % t, ["-DFP6MI_FORMAT=%d" % t]) for t in FORMAT_TAGS]
OBJ_DIR = os.path.join(HERE, "csrc", "obj")
OUTPUT = os.path.join(HERE, "libfp6mi.so")
# measurement aid for the benchmark (a read-only streaming kernel); not linked into the engine
PROBE_SOURCES = [os.path.join(HERE, "csrc", "stream_probe.hip")]
PROBE_OUTPUT = os.path.join(HERE, "libfp6mi_probe.so")


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the FPx engine cannot be built without the ROCm compiler")


def _hipcc(args, what, verbose):
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
           # packed FP32 VALU forms are kept out of the generated code on this hardware pool
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I" + os.path.join(ROOT, "include")] + args
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        sys.stderr.write("\n".join(l for l in (res.stdout + res.stderr).splitlines() if "packed-fp32-ops" not in l) + "\n")
    if res.returncode != 0:
        raise RuntimeError("hipcc failed building " + what)


def _compile(sources, output, verbose):
    _hipcc(["-shared"] + sources + ["-o", output + ".tmp"], os.path.basename(output), verbose)
    os.replace(output + ".tmp", output)
    return output


def _compile_library(verbose):
    """Every translation unit of libfp6mi.so to an object (in parallel: the kernels of each format take most of the time),
    then one link."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, o) for _, o, _ in UNITS]

    def one(unit):
        src, obj, flags = unit
        _hipcc(["-c", os.path.join(HERE, "csrc", src), "-o", os.path.join(OBJ_DIR, obj)] + flags, obj, verbose)
    with ThreadPoolExecutor(max_workers=min(len(UNITS), os.cpu_count() or 1)) as pool:
        list(pool.map(one, UNITS))
    _hipcc(["-shared"] + objs + ["-o", OUTPUT + ".tmp"], "libfp6mi.so", verbose)
    os.replace(OUTPUT + ".tmp", OUTPUT)
    return OUTPUT


def build_torch_extension(verbose=False):
    """Compiles csrc/torch_binding.cpp (a host-only translation unit: g++, torch's headers, the C ABI) into
    _fp6mi_torch.so next to libfp6mi.so, which must exist."""
    import sysconfig

    from torch.utils import cpp_extension as ce
    import torch

    out = os.path.join(HERE, "_fp6mi_torch.so")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_fp6mi_torch",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch.compiled_with_cxx11_abi())]
    cmd += ["-I" + p for p in ce.include_paths()] + ["-I" + sysconfig.get_paths()["include"], "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include")]
    cmd += [os.path.join(HERE, "csrc", "torch_binding.cpp")]
    libdirs = ce.library_paths()
    cmd += ["-L" + p for p in libdirs] + ["-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-L" + HERE, "-lfp6mi", "-Wl,-rpath,$ORIGIN"]
    cmd += ["-Wl,-rpath," + p for p in libdirs] + ["-o", out + ".tmp"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
    if res.returncode != 0:
        raise RuntimeError("g++ failed building _fp6mi_torch.so")
    os.replace(out + ".tmp", out)
    return out


def build(verbose=False):
    """Compiles every HIP/C++ source for gfx950 into libfp6mi.so and libfp6mi_probe.so, then the torch extension over the C
    ABI (always recompiles)."""
    _compile(PROBE_SOURCES, PROBE_OUTPUT, verbose)
    lib = _compile_library(verbose)
    build_torch_extension(verbose)
    return lib


if __name__ == "__main__":
    print(build(verbose=True))
