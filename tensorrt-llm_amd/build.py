"""Builds libwoq.so (HIP kernels + C ABI) for gfx950 in-tree, next to this file.

    python tensorrt-llm_amd/build.py [--jobs N]

hipcc cross-compiles without a GPU.  Every translation unit is compiled on its own (in parallel)
and the objects are linked into one shared library with no dependency on torch.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.environ.get("WOQ_OBJ_DIR") or os.path.join(HERE, "build")
LIB = os.environ.get("WOQ_LIB_OUT") or os.path.join(HERE, "libwoq.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 ops are switched off for all device code (compiler-generated v_pk_*_f32 forms have
# produced wrong results on this hardware pool)
# Kernels whose arguments are plain scalars find the first fourteen dwords of them in SGPRs when a wavefront
# starts (kernel-argument preloading) instead of fetching them with scalar loads, 0.2-0.3 us per dependent
# batch; kernels that take a struct by value are unaffected.
DEVICE_FLAGS = ["--offload-arch=" + ARCH, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-mllvm", "-amdgpu-kernarg-preload-count=16"]
COMMON = ["-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
          "-ffp-contract=off"]
# Per-file additions.  The skinny-M kernel reads its MFMA results with VALU instructions every
# group: keep those accumulators in the architectural VGPRs instead of copying them out of AGPRs.
PER_FILE = {"skinny_": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def sources():
    out = []
    for root, _, files in os.walk(CSRC):
        for f in sorted(files):
            if f.endswith((".hip", ".cpp")):
                out.append(os.path.join(root, f))
    return sorted(out)


def _headers_mtime() -> float:
    newest = 0.0
    for root, _, files in os.walk(os.path.dirname(HERE)):
        if os.sep + "build" in root or os.sep + "." in root:
            continue
        for f in files:
            if f.endswith(".h"):
                newest = max(newest, os.path.getmtime(os.path.join(root, f)))
    return newest


_ONLY_CHANGED = False  # --changed: skip a translation unit whose object is newer than it and every header


def _compile(src: str) -> str:
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    obj = os.path.join(OBJ, rel + ".o")
    if _ONLY_CHANGED and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), _headers_mtime()):
        return obj
    extra = os.environ.get("WOQ_EXTRA_FLAGS", "").split()
    for prefix, flags in PER_FILE.items():
        if os.path.basename(src).startswith(prefix):
            extra = extra + flags
    cmd = [HIPCC, "-x", "hip"] + DEVICE_FLAGS + COMMON + extra + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "unknown to the target"  # host pass does not know the device-only feature flag
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l and "'-packed-fp32-ops'" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_lib(jobs: int | None = None, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, os.cpu_count() or 1)
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built %s from %d translation units" % (LIB, len(srcs)))
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=None)
    ap.add_argument("--changed", action="store_true", help="recompile only what changed (development)")
    ap.add_argument("--timeline", action="store_true",
                    help="a second library, libwoq_timeline.so, whose row decode kernel records per-wavefront time "
                         "stamps (-DWOQ_TIMELINE; objects in build_timeline/): for `bench.py --mode timeline`")
    a = ap.parse_args()
    _ONLY_CHANGED = a.changed
    if a.timeline:
        OBJ = os.path.join(HERE, "build_timeline")
        LIB = os.path.join(HERE, "libwoq_timeline.so")
        DEVICE_FLAGS = DEVICE_FLAGS + ["-DWOQ_TIMELINE"]
    build_lib(a.jobs)
