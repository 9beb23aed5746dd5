"""Builds libmi355_qlinear.so for gfx950 with hipcc (one object per translation unit, in parallel).

Usage:  python swift-mlx-lm_amd/build.py [--force] [-j N] [--timeline]
The library is written to swift-mlx-lm_amd/lib/ (git-ignored, travels with the tree).
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libmi355_qlinear.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


# Translation units whose kernels must not spill vector registers (beyond the count of the build the GPU tests ran on):
# the wide-tile prefill kernel issues its weight loads as hand-written instructions with hand-counted waits.
SPILL_GUARDED = {"gemm_wide_bf16.hip": 2, "gemm_wide_f16.hip": 2}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _deps_mtime():
    return max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC)
               if f.endswith((".h", ".inl"))) if os.path.isdir(CSRC) else 0.0


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, src + ".o")
    srcp = os.path.join(CSRC, src)
    inc = os.path.join(HERE, "..", "include")
    newest = max(os.path.getmtime(srcp), _deps_mtime(), *(os.path.getmtime(os.path.join(inc, h)) for h in os.listdir(inc)))
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest:
        return obj
    cmd = [HIPCC, *FLAGS, "-x", "hip", "-c", srcp, "-o", obj]
    guarded = src in SPILL_GUARDED
    if guarded:
        cmd.insert(-4, "-Rpass-analysis=kernel-resource-usage")      # remarks only: the code is the same
    r = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the packed-fp32 feature name; that one line is harmless
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "kernel-resource-usage" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if guarded:
        name, worst = "", []
        for line in r.stderr.splitlines():
            if "Function Name:" in line:
                name = line.split("Function Name:")[1].split("[")[0].strip()
            elif "VGPRs Spill:" in line:
                n = int(line.split("VGPRs Spill:")[1].split("[")[0])
                if n > SPILL_GUARDED[src]:
                    worst.append(f"{name}: {n}")
        if worst:
            os.remove(obj)
            raise RuntimeError(f"{src}: vector registers spilled beyond the {SPILL_GUARDED[src]} of the tested build -- " +
                               "; ".join(worst) + ".  This kernel's hand-written loads deliver their data after the statement "
                               "that issued them: a target register the compiler has saved and reused is overwritten when the "
                               "load lands (a memory fault at run time).  Shorten what lives across its K loop.")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_timeline(jobs: int | None = None) -> str:
    """Measurement build: the library with per-workgroup time stamps in the decode rows kernel
    (-DMI355Q_GEMV_TIMELINE), written beside the product library as libmi355_qlinear_timeline.so.
    Used by decode_timeline.py only; the product library carries none of it."""
    global OBJ, LIB, FLAGS
    saved = (OBJ, LIB, FLAGS)
    try:
        OBJ = os.path.join(HERE, "build_timeline")
        LIB = os.path.join(LIBDIR, "libmi355_qlinear_timeline.so")
        FLAGS = FLAGS + ["-DMI355Q_GEMV_TIMELINE"]
        return build(force=False, jobs=jobs)
    finally:
        OBJ, LIB, FLAGS = saved


def build(force: bool = False, jobs: int | None = None) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    # objects compiled with other flags are stale whatever their age
    stamp = os.path.join(OBJ, "flags.txt")
    flags_now = " ".join(FLAGS)
    if not os.path.exists(stamp) or open(stamp).read() != flags_now:
        force = True
    jobs = jobs or min(8, os.cpu_count() or 4)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    with open(stamp, "w") as f:
        f.write(flags_now)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    ap.add_argument("--timeline", action="store_true", help="the measurement build with per-workgroup time stamps (decode_timeline.py)")
    a = ap.parse_args()
    print(build_timeline(jobs=a.j) if a.timeline else build(force=a.force, jobs=a.j))
