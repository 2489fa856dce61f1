"""Builds the C-ABI operator library (libc_runtime_api.so) for gfx950 with hipcc, in-tree.

    python -m tsplit_amd.build            # incremental
    python -m tsplit_amd.build --force    # recompile everything

Also builds the host-only pool test library used by the CPU tests.
"""
import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "_obj")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libc_runtime_api.so")
POOL_TEST_LIB = os.path.join(LIBDIR, "libtsplit_pool_host.so")

HIPCC = os.environ.get("HIPCC", shutil.which("hipcc") or "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 code generation is switched off for every device object of this library
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unknown-warning-option"]
FLAGS += os.environ.get("TSPLIT_EXTRA_HIPCC_FLAGS", "").split()


def _sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")) and not f.startswith("pool_capi"))


def _headers_mtime():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(HERE, "..", "include", "c_runtime_api.h"))
    return max(os.path.getmtime(h) for h in hs)


def _compile(src, force, hmtime):
    obj = os.path.join(OBJ, src + ".o")
    path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), hmtime):
        return obj, False
    cmd = [HIPCC, *FLAGS, "-x", "hip", "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj, True


def build(force=False, jobs=8, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    hmtime = _headers_mtime()
    srcs = _sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda s: _compile(s, force, hmtime), srcs))
    objs = [o for o, _ in results]
    if force or any(c for _, c in results) or not os.path.exists(LIB):
        cmd = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", LIB]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    # host-only pool library for the CPU tests (plain g++, no HIP)
    pool_src = os.path.join(CSRC, "pool_capi.cpp")
    if os.path.exists(pool_src):
        need = force or not os.path.exists(POOL_TEST_LIB) or \
            os.path.getmtime(POOL_TEST_LIB) < max(os.path.getmtime(pool_src), os.path.getmtime(os.path.join(CSRC, "pool.h")))
        if need:
            r = subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", pool_src, "-o", POOL_TEST_LIB],
                               capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"g++ failed on pool_capi.cpp:\n{r.stderr}")
    # stand-alone measurement programs (csrc/probes/*.hip -> lib/<name>)
    probes = os.path.join(CSRC, "probes")
    for f in sorted(os.listdir(probes)) if os.path.isdir(probes) else []:
        if not f.endswith(".hip"):
            continue
        exe, src = os.path.join(LIBDIR, f[:-4]), os.path.join(probes, f)
        if force or not os.path.exists(exe) or os.path.getmtime(exe) < os.path.getmtime(src):
            r = subprocess.run([HIPCC, *[x for x in FLAGS if x != "-fPIC"], "-Wno-unused-value", src, "-o", exe], capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"hipcc failed on probes/{f}:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} ({sum(c for _, c in results)}/{len(srcs)} objects recompiled)")
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=8)
    a = ap.parse_args()
    build(a.force, a.j)
