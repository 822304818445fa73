"""Builds the native libraries of this package with hipcc / g++ (gfx950 only).

    python intel-extension-for-tensorflow_amd/build.py [--jobs N]

Outputs (next to this file, git-ignored):
    lib/libitexhip.so        HIP kernels + the C ABI declared in include/itexhip.h
    lib/libitex_amd.so       the TensorFlow PluggableDevice kernel plugin (TF_InitKernel), if its
                             sources are present
"""
import argparse
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
PLUGIN = os.path.join(HERE, "plugin")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "build")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fno-fast-math", "-fno-gpu-flush-denormals-to-zero",
    # no packed-fp32 instructions in device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm", "-I", INCLUDE, "-I", CSRC,
]
CXX = os.environ.get("CXX", "g++")
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-Wall", "-I", INCLUDE,
             "-I", PLUGIN]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout)
        raise RuntimeError("build step failed: " + " ".join(cmd[:3]))
    return proc.stdout


def _has_untracked_asm(src):
    """True for the translation units that hold memory instructions written as inline assembly (the tile kernels)."""
    return os.path.basename(src).startswith("qgemm_tile_")


def device_assembly_of(src):
    """Where the compile step leaves the device assembly of a translation unit with inline-assembly memory instructions."""
    stem = os.path.splitext(os.path.basename(src))[0]
    return os.path.join(OBJ, stem + "-hip-amdgcn-amd-amdhsa-gfx950.s")


def _compile_hip(src):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    keep = ["-save-temps=obj"] if _has_untracked_asm(src) else []
    out = _run([HIPCC] + HIP_FLAGS + keep + ["-c", src, "-o", obj])
    if keep:   # only the device assembly is wanted from the intermediate files
        stem = os.path.splitext(os.path.basename(src))[0]
        for f in glob.glob(os.path.join(OBJ, stem + "-h*")) + glob.glob(os.path.join(OBJ, stem + ".hip-hip-*")):
            if f != device_assembly_of(src):
                os.remove(f)
    # the host pass does not know the packed-fp32 feature name; that warning is expected
    out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if out:
        sys.stderr.write(out + "\n")
    return obj


def check_inline_asm_hazards(asm_files, verbose=True):
    """The compiler neither counts the inline-assembly loads of the tile kernels in its wait counts nor gives their
    assembly stores hazard wait states; csrc/check_asm_hazards.py proves on the compiled device assembly that the
    hand-written waits cover every path.  A finding fails the build: the library is not linked."""
    import contextlib
    import importlib.util
    import io
    spec = importlib.util.spec_from_file_location("check_asm_hazards", os.path.join(CSRC, "check_asm_hazards.py"))
    chk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(chk)
    log = io.StringIO()
    with contextlib.redirect_stdout(log):
        flagged = sum(chk.check_file(f) for f in asm_files)
    if flagged:
        sys.stderr.write(log.getvalue())
        raise RuntimeError("inline-assembly hazard check failed: %d finding(s) in the tile kernels' device assembly" % flagged)
    if verbose:
        print("inline-assembly hazard check: %d assembly files clean" % len(asm_files))


def build(jobs=8, verbose=True):
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    hip_srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile_hip, hip_srcs))
    check_inline_asm_hazards([device_assembly_of(f) for f in hip_srcs if _has_untracked_asm(f)], verbose)
    libitexhip = os.path.join(LIB, "libitexhip.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", libitexhip] + objs)
    if verbose:
        print("built", os.path.relpath(libitexhip, ROOT))
    built = [libitexhip]
    plugin_srcs = sorted(glob.glob(os.path.join(PLUGIN, "*.cc")))
    if plugin_srcs:
        libplugin = os.path.join(LIB, "libitex_amd.so")
        # TF_* symbols stay undefined: the TensorFlow runtime (or the mock host of the tests) provides them
        _run([CXX] + CXX_FLAGS + ["-shared", "-o", libplugin] + plugin_srcs +
             ["-L", LIB, "-litexhip", "-Wl,-rpath,$ORIGIN", "-pthread"])
        if verbose:
            print("built", os.path.relpath(libplugin, ROOT))
        built.append(libplugin)
    return built


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=8)
    build(ap.parse_args().jobs)
