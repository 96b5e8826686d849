"""Builds libspamm_gfx950.so (HIP kernels + C ABI) in-tree with hipcc.

Usage: ``python -m cuspamm_amd.build`` (or ``build_library()`` from Python).
The library is cross-compiled for gfx950 and needs no GPU to build.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libspamm_gfx950.so")
DEV_LIB_PATH = os.path.join(HERE, "libspamm_dev_gfx950.so")   # measurement aids (csrc/dev_probe.hip), not the engine
MAIN_PATH = os.path.join(HERE, "spamm_main")     # the reference's main() on top of the C ABI (csrc/spamm_main.cpp)

SOURCES = ["kernels_normmap.hip", "kernels_gate.hip", "kernels_gemm.hip", "kernels_tau.hip", "kernels_tools.hip",
           "spamm_api.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops is switched off on purpose: the compiler must not form
# v_pk_{add,mul,fma}_f32 from the norm accumulation.
CFLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# kernels_gemm.hip only.  M0 is listed as clobbered by its global->LDS loads and clang remarks on every
# instance that M0 is reserved (it never allocates it anyway).  The ticket of the workgroups that stay is
# drawn by one lane with a returning atomic that is asked for early and looked at late; the compiler's
# rewrite of atomics in divergent code (one lane adds for all, then a broadcast) would wait for it at once.
GEMM_FLAGS = ["-Wno-inline-asm", "-mllvm", "-amdgpu-atomic-optimizer-strategy=None"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "packed-fp32-ops" not in line or "is not a recognized feature" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _check_no_scratch(log, src):
    """The GEMM keeps 256 accumulator registers per lane; a compiler version or an edit that
    makes it spill them to scratch memory costs a factor of several, so refuse such a build."""
    import re
    name = None
    for line in log.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name and "k_gemm" in name and int(m.group(1)) != 0:
            raise RuntimeError("%s: kernel %s spills %s bytes/lane to scratch" % (src, name, m.group(1)))


def build_library(verbose=False):
    """Compiles every HIP source and links the shared library. Always rebuilds."""
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        extra = ["-Rpass-analysis=kernel-resource-usage"] + GEMM_FLAGS if src == "kernels_gemm.hip" else []
        log = _run([HIPCC] + CFLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj])
        if extra:
            _check_no_scratch(log, src)
            keep, skip = [], 0
            for line in log.splitlines():          # drop the remarks and the source excerpts printed under them
                if "remark:" in line:
                    skip = 2
                elif skip and (line.lstrip().startswith("|") or "|" in line[:8]):
                    skip -= 1
                else:
                    skip = 0
                    keep.append(line)
            log = "\n".join(keep)
        return log

    with ThreadPoolExecutor(max_workers=4) as ex:
        logs = list(ex.map(compile_one, zip(SOURCES, objs)))
    logs.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs))
    logs.append(_run([HIPCC] + CFLAGS + ["-shared", os.path.join(CSRC, "dev_probe.hip"), "-o", DEV_LIB_PATH]))
    logs.append(_run([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-Wall", os.path.join(CSRC, "spamm_main.cpp"), "-o", MAIN_PATH,
                      "-L" + HERE, "-lspamm_gfx950", "-Wl,-rpath,$ORIGIN"]))
    if verbose:
        for text in logs:
            if text.strip():
                print(text)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
