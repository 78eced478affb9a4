"""Builds ``libfsta.so`` (HIP kernels + C ABI) for gfx950 with hipcc.

    python -m fstattention_amd.build

The library is written next to this file so that it travels with the source
tree; nothing is installed.  hipcc cross-compiles, so no GPU is needed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libfsta.so")
OBJ_DIR = os.path.join(PKG_DIR, "csrc", "_obj")

SOURCES = [
    "fsta_capi.hip",
    "fsta_precompute.hip",
    "fsta_tree_order.hip",
    "fsta_tree_build.hip",
    "fsta_merge.hip",
    "fsta_attention_generic.hip",
    "fsta_attention_mfma.hip",
    "fsta_attention_mfma16.hip",
    "fsta_attention_prefix.hip",
    "fsta_attention_stream.hip",
    "fsta_roofline.hip",
]

# packed-fp32 VALU forms are switched off for device code on purpose
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-option-ignored",
    "-Rpass-analysis=kernel-resource-usage",
]

# Kernels of these sources must keep everything in registers: a private array the compiler leaves
# in scratch memory, or a spill, is reloaded through the same vmcnt queue their gather rings count on.
NO_SCRATCH = ("fsta_attention_mfma16.hip", "fsta_attention_mfma.hip", "fsta_attention_prefix.hip",
              "fsta_attention_stream.hip", "fsta_attention_generic.hip")


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, proc.stderr))
    return proc.stderr


def _split_resource_remarks(stderr: str):
    """hipcc's -Rpass-analysis=kernel-resource-usage remarks -> ({kernel: {field: int}}, the other lines)."""
    usage, rest, current, skip = {}, [], None, 0
    for line in stderr.splitlines():
        if skip:                      # the two source-quote lines clang prints under the first remark of a kernel
            skip -= 1
            continue
        if "[-Rpass-analysis=kernel-resource-usage]" in line:
            body = line.split("remark:", 1)[1].rsplit("[-Rpass", 1)[0].strip()
            key, _, val = body.rpartition(":")
            if key.strip() == "Function Name":
                current = usage.setdefault(val.strip(), {})
                skip = 2
            elif current is not None:
                try:
                    current[key.strip()] = int(val)
                except ValueError:
                    pass
            continue
        rest.append(line)
    return usage, "\n".join(rest)


TIMELINE_LIB_PATH = os.path.join(PKG_DIR, "libfsta_timeline.so")


def build_library(verbose: bool = True, jobs: int | None = None, timeline: bool = False) -> str:
    """Compiles every source and links ``libfsta.so``; always rebuilds.  ``timeline=True`` builds the
    instrumented variant ``libfsta_timeline.so`` instead (``-DFSTA_TIMELINE``: the matrix-core kernel notes
    cycle stamps, see ``fstattention_amd/timeline.py``); the regular library is left alone."""
    hipcc = _hipcc()
    obj_dir = OBJ_DIR + ("_timeline" if timeline else "")
    lib_path = TIMELINE_LIB_PATH if timeline else LIB_PATH
    extra = ["-DFSTA_TIMELINE"] if timeline else []
    sources = SOURCES
    os.makedirs(obj_dir, exist_ok=True)
    jobs = jobs or min(len(sources), os.cpu_count() or 1, 16)

    def compile_one(src):
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        warn = _run([hipcc, *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj])
        return obj, warn

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(compile_one, sources))
    for (obj, warn), src in zip(results, sources):
        usage, warn = _split_resource_remarks(warn)
        if src in NO_SCRATCH and not timeline:
            bad = [(name, u) for name, u in usage.items() if u.get("ScratchSize [bytes/lane]", 0)]
            if bad:
                raise RuntimeError(f"{src}: kernels using scratch memory: " +
                                   ", ".join(f"{n} ({u['ScratchSize [bytes/lane]']} B/lane)" for n, u in bad))
        # hipcc's host pass does not know the device-only feature name: not a problem
        warn = "\n".join(l for l in warn.splitlines() if "packed-fp32-ops" not in l)
        if verbose and warn.strip():
            sys.stderr.write(warn + "\n")
    objs = [o for o, _ in results]
    tmp = lib_path + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, lib_path)
    if verbose:
        print(f"built {lib_path} ({os.path.getsize(lib_path)} bytes)")
    return lib_path


TORCH_OPS_PATH = os.path.join(PKG_DIR, "_fsta_torch.so")


def build_torch_ops(verbose: bool = True) -> str:
    """Compiles ``csrc/fsta_torch_binding.cpp`` (host code: the ``torch.ops.fsta`` registration on top of
    the C ABI) with the host compiler against this interpreter's torch and links it to ``libfsta.so``."""
    import torch
    from torch.utils import cpp_extension as ce
    cxx = os.environ.get("CXX") or shutil.which("g++")
    if not cxx:
        raise RuntimeError("g++ not found (set CXX)")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    includes = [f"-I{d}" for d in ce.include_paths("cuda")]
    tmp = TORCH_OPS_PATH + ".tmp"
    _run([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
          f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations",
          *includes, os.path.join(CSRC, "fsta_torch_binding.cpp"), "-o", tmp,
          f"-L{torch_lib}", "-lc10", "-ltorch_cpu", "-ltorch_hip", "-lc10_hip", "-ltorch",
          f"-L{PKG_DIR}", "-l:libfsta.so", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"])
    os.replace(tmp, TORCH_OPS_PATH)
    if verbose:
        print(f"built {TORCH_OPS_PATH} ({os.path.getsize(TORCH_OPS_PATH)} bytes)")
    return TORCH_OPS_PATH


if __name__ == "__main__":
    if "--timeline" in sys.argv[1:]:
        build_library(timeline=True)
    else:
        build_library()
        build_torch_ops()
