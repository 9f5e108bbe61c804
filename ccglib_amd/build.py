"""Builds libccglib_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in tree.

    python -m ccglib_amd.build            # compile what changed, link
    python -m ccglib_amd.build --force    # recompile everything
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(HERE, "libccglib_amd.so")
# (gemm_mfma.hip is compiled in parts, one per input type, so that they build in parallel)
SOURCES = ["capi.hip", "gemm_mfma_f16.hip", "gemm_mfma_bf16.hip", "gemm_mfma_f32.hip",
           "gemm_mfma_fp8.hip", "gemm_mfma_int1.hip", "gemm_mfma_dispatch.hip", "gemm_int1.hip",
           "transpose.hip", "packing.hip"]
HEADERS = [os.path.join(CSRC, "common.h"), os.path.join(CSRC, "gemm_device.h"),
           os.path.join(CSRC, "gemm_mfma.hip"), os.path.join(CSRC, "gemm_mfma_wide.h"),
           os.path.join(os.path.dirname(HERE), "include", "ccglib_amd.h")]

# Packed-fp32 instruction selection is switched off for all device code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _defines():
    """Build options taken from the environment: CCGLIB_AMD_STATIC_SCRATCH_BYTES, the size
    of the static device array of ccglib_pipeline_run_static (default in the header)."""
    v = os.environ.get("CCGLIB_AMD_STATIC_SCRATCH_BYTES")
    return ["-DCCGLIB_AMD_STATIC_SCRATCH_BYTES=((size_t)%d)" % int(v)] if v else []


def _hipcc():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if not force and not _stale(obj, [path] + HEADERS):
        return obj, ""
    cmd = [_hipcc()] + HIPCC_FLAGS + _defines() + ["-Rpass-analysis=kernel-resource-usage", "-c", path,
                                                   "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    lines = (r.stdout + r.stderr).splitlines()
    kept, skip = [], 0
    for l in lines:      # (the remarks, each with its source line and caret, stay out of the log)
        if "kernel-resource-usage" in l:
            skip = 2
        elif skip and (l.lstrip()[:1].isdigit() or l.strip().startswith("|")):
            skip -= 1
        elif "packed-fp32-ops" not in l:
            kept.append(l)
            skip = 0
    log = "\n".join(kept)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    _no_scratch_in_gemm_kernels(src, lines)
    return obj, log


def _no_scratch_in_gemm_kernels(src, remarks):
    """The MFMA GEMM kernels wait for their copies with explicit `s_waitcnt vmcnt(n)` counts,
    which only hold while the compiler adds no memory instructions of its own inside the K
    loop. The compiler's resource remarks say whether a kernel spills registers to scratch
    memory. The one-wave-per-SIMD kernels (complex_gemm_mfma_wide) run at the edge of the
    register file and must not spill at all: the build stops if one does. Of the others, the
    1-bit 128 x 128 kernel spills four values at set-up and reloads them where a block moves
    to its next C tile (the compiler waits for all memory operations there); anything beyond
    those few bytes stops the build as well."""
    name = None
    for l in remarks:
        if "Function Name:" in l:
            name = l.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in l and name and "complex_gemm_mfma" in name:
            size = int(l.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            if size > (0 if "complex_gemm_mfma_wide" in name else 32):
                os.remove(os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o"))
                raise RuntimeError("%s: kernel %s spills %d bytes per lane to scratch memory; its "
                                   "explicit vmcnt counts would not hold" % (src, name, size))


def build(force=False, verbose=False):
    """Compile every HIP source for gfx950 and link the shared library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, log in results:
            if log.strip():
                print(log)
    if force or _stale(LIB_PATH, objs):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
