"""Builds libmoe_hip.so (the HIP kernels + C ABI) for gfx950 with hipcc.

    python moe-explore_amd/build.py [--jobs N] [--force]
    python moe-explore_amd/build.py --ablate N --out /some/dir/libmoe_hip_ablate.so

The second form builds a diagnostic copy of the library whose GEMM kernels leave parts of
their K loop out (-DMOE_ABLATE=N, see csrc/gemm_mfma_dma.hip and csrc/gemm_kgrouped.hip): wrong
results, used only to time what a K step spends on what (MOE_HIP_LIB=<that file> bench.py
--only ablation).  It never touches moe_explore/libmoe_hip.so.

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


def build_ablation(mask, out):
    """Diagnostic library: the two GEMM sources compiled with -DMOE_ABLATE=mask, linked with the
    product build's other objects into `out` (which must not be the product library)."""
    out = os.path.abspath(out)
    assert out != os.path.abspath(LIB), "an ablation build never replaces the product library"
    build(verbose=False)
    os.makedirs(os.path.dirname(out), exist_ok=True)
    tmp = out + ".objs"
    os.makedirs(tmp, exist_ok=True)
    swapped = ("gemm_mfma_dma", "gemm_kgrouped")
    objs = [os.path.join(BUILD, f[:-4] + ".o") for f in sorted(os.listdir(CSRC))
            if f.endswith(".hip") and f[:-4] not in swapped]
    for name in swapped:
        obj = os.path.join(tmp, name + ".o")
        _, rc, log = _compile(os.path.join(CSRC, name + ".hip"), obj, [f"-DMOE_ABLATE={int(mask)}"])
        if rc != 0:
            print(log, file=sys.stderr)
            raise RuntimeError("hipcc failed")
        objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out,
           "-Wl,-rpath,/opt/rocm/lib", "-Wl,--no-undefined"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    shutil.rmtree(tmp, ignore_errors=True)
    if r.returncode != 0:
        print(r.stdout + r.stderr, file=sys.stderr)
        raise RuntimeError("link failed")
    print(f"[build] ablation {mask}: {out}")
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=None)
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--ablate", type=int, default=None, metavar="MASK",
                    help="build a diagnostic library with -DMOE_ABLATE=MASK instead (needs --out)")
    ap.add_argument("--out", default=None, help="path of the ablation library")
    a = ap.parse_args()
    if a.ablate is not None:
        if not a.out:
            ap.error("--ablate needs --out")
        build_ablation(a.ablate, a.out)
    else:
        build(jobs=a.jobs, force=a.force)
