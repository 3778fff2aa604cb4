"""Builds libmoe_hip.so (the HIP kernels + C ABI) for gfx950 with hipcc.

    python moe-explore_amd/build.py [--jobs N] [--force]

Each csrc/*.hip is compiled to an object under build/ and the objects are linked
into moe_explore/libmoe_hip.so.  Nothing is compiled at import time: the Python
package only loads the library this script leaves behind.
"""
import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "moe_explore", "libmoe_hip.so")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
CXXFLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-munsafe-fp-atomics",
    # packed-fp32 VALU forms are kept out of generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _compile(src, obj, extra):
    cmd = [HIPCC, *CXXFLAGS, *extra, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, r.returncode, (r.stdout + r.stderr)


def build(jobs=None, force=False, verbose=True, extra=()):
    os.makedirs(BUILD, exist_ok=True)
    sources = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(HERE, "..", "include", "moe_hip.h"))
    todo, objs = [], []
    for f in sources:
        src = os.path.join(CSRC, f)
        obj = os.path.join(BUILD, f[:-4] + ".o")
        objs.append(obj)
        if force or not _newer(obj, [src, *headers]):
            todo.append((src, obj))
    jobs = jobs or min(8, os.cpu_count() or 1)
    failed = False
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, rc, out in pool.map(lambda so: _compile(so[0], so[1], list(extra)), todo):
            errs = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
            if rc != 0:
                failed = True
                print(f"[build] FAILED {os.path.basename(src)}\n" + "\n".join(errs), file=sys.stderr)
            elif verbose:
                print(f"[build] compiled {os.path.basename(src)}")
    if failed:
        raise RuntimeError("hipcc failed")
    if todo or force or not os.path.exists(LIB):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB,
               "-Wl,-rpath,/opt/rocm/lib", "-Wl,--no-undefined"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            print(r.stdout + r.stderr, file=sys.stderr)
            raise RuntimeError("link failed")
        if verbose:
            print(f"[build] linked {LIB}")
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=None)
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args()
    build(jobs=a.jobs, force=a.force)
