"""Builds the two shared libraries of the MI355X backend with hipcc (gfx950 only).

  lib/libdiopi_impl.so   DIOPI operator entry points + hand-written HIP kernels.
                         Leaves the diopirt callbacks undefined: DIPU (or lib/libdipu_amd_rt.so)
                         provides them at load time.
  lib/libdipu_amd_rt.so  dipu::devapis over HIP, stream/event pools, caching allocators,
                         diopirt callbacks and the C facade declared in include/dipu_amd/runtime.h.

Usage: python build.py [-j N] [--only impl|rt]
"""
import argparse
import concurrent.futures
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")

ARCH = "gfx950"
# packed-fp32 VALU forms are switched off for all device code on this platform
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON = ["-O3", "-fPIC", "-std=c++17", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
          f"--offload-arch={ARCH}", f"-I{INCLUDE}"] + DEVICE_FLAGS

TARGETS = {
    "impl": {
        "dir": os.path.join(HERE, "csrc", "diopi_impl"),
        "out": os.path.join(LIB_DIR, "libdiopi_impl.so"),
        "link": [],
    },
    "rt": {
        "dir": os.path.join(HERE, "csrc", "runtime"),
        "out": os.path.join(LIB_DIR, "libdipu_amd_rt.so"),
        "link": [],
    },
}


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def sources(d):
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith((".hip", ".cpp")))


# Kernels whose K loop is inline assembly over fixed physical registers (accumulators and operand fragments the
# compiler knows only as clobbered): they are correct only while the compiler keeps nothing of its own in scratch
# memory around that text, so a build in which one of them uses scratch fails. (Scalar registers the compiler
# parks in lanes of a vector register are not scratch: they cost a lane write and a lane read, no memory access.)
NO_SCRATCH_KERNELS = {"gemm.hip": ("gemmMfma4WaveKernel",)}


def scratch_users(remarks, names):
    """Kernels (mangled names holding one of `names`) whose resource-usage remark reports scratch or spilled vector registers."""
    bad, current = [], None
    for line in remarks.splitlines():
        if "remark:" not in line:
            continue
        text = line.split("remark:", 1)[1].strip()
        if text.startswith("Function Name:"):
            fn = text.split(":", 1)[1].split("[")[0].strip()
            current = fn if any(n in fn for n in names) else None
        elif current and (text.startswith("ScratchSize") or text.startswith("VGPRs Spill")):
            if int(text.split(":", 1)[1].split("[")[0].strip()) != 0:
                bad.append(f"{current}: {text.split('[-R')[0].strip()}")
    return bad


def compile_one(src, obj):
    watch = NO_SCRATCH_KERNELS.get(os.path.basename(src))
    extra = ["-Rpass-analysis=kernel-resource-usage"] if watch else []
    cmd = [hipcc()] + COMMON + extra + ["-x", "hip", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    stderr = r.stderr
    rc = r.returncode
    if watch:
        bad = scratch_users(stderr, watch)
        seen = any(n in stderr for n in watch)
        # a remark is followed by an echo of the source line ("  806 | __global__ ...") and a caret line
        echo = re.compile(r"^\s*(\d+\s*)?\|")
        stderr = "\n".join(l for l in stderr.splitlines() if "kernel-resource-usage" not in l and not echo.match(l))
        if rc == 0 and not seen:
            stderr += f"\n{os.path.basename(src)}: no resource-usage remark for {watch}: the scratch check did not run"
            rc = 1
        if bad:
            stderr += "\n" + "\n".join("uses scratch memory around a hand-placed register loop: " + b for b in bad)
            rc = 1
    err = "\n".join(l for l in stderr.splitlines() if "packed-fp32-ops" not in l)
    return src, rc, err


def build(only=None, jobs=None):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    names = [only] if only else list(TARGETS)
    work = []
    for name in names:
        t = TARGETS[name]
        for src in sources(t["dir"]):
            obj = os.path.join(OBJ_DIR, name + "_" + os.path.basename(src) + ".o")
            work.append((name, src, obj))
    failed = False
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = [ex.submit(compile_one, src, obj) for _, src, obj in work]
        for f in concurrent.futures.as_completed(futs):
            src, rc, err = f.result()
            if err.strip():
                sys.stderr.write(err + "\n")
            if rc != 0:
                sys.stderr.write(f"FAILED: {src}\n")
                failed = True
    if failed:
        raise RuntimeError("hipcc compilation failed")
    for name in names:
        t = TARGETS[name]
        objs = [obj for n, _, obj in work if n == name]
        cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", t["out"]] + objs + t["link"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stderr)
            raise RuntimeError(f"link failed: {t['out']}")
    return [TARGETS[n]["out"] for n in names]


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=None)
    ap.add_argument("--only", choices=list(TARGETS), default=None)
    a = ap.parse_args()
    for out in build(a.only, a.j):
        print("built", out)
