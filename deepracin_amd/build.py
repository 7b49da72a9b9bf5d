"""Build libdeepracin.so (host graph code + hand-written gfx950 HIP kernels) in-tree with hipcc.

    python -m deepracin_amd.build            # incremental
    python -m deepracin_amd.build --force    # recompile everything

The library lands in deepracin_amd/lib/libdeepracin.so; objects in deepracin_amd/lib/obj/.
hipcc cross-compiles for gfx950, so this works on a machine without a GPU.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libdeepracin.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-fPIC", "-std=c++17", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(CSRC, "device"),
          "-I" + os.path.join(CSRC, "host"), "-Wall", "-Wno-unused-function"]
# Packed-fp32 VALU forms are kept out of the generated code on purpose.
# The first 16 dwords of every kernel's arguments arrive in SGPRs with the wave instead of through a scalar load at
# its start (gfx950 kernarg preload): about 0.1 us off each of the 19-23 launches of a batch-1 pass.
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def sources():
    out = []
    for sub in ("host", "device"):
        d = os.path.join(CSRC, sub)
        for f in sorted(os.listdir(d)):
            if f.endswith(".cpp") or f.endswith(".hip"):
                out.append(os.path.join(d, f))
    return out


def headers_mtime():
    newest = 0.0
    for d in (os.path.join(ROOT, "include"), os.path.join(CSRC, "host"), os.path.join(CSRC, "device")):
        for f in os.listdir(d):
            if f.endswith((".h", ".hpp")):
                newest = max(newest, os.path.getmtime(os.path.join(d, f)))
    return newest


def compile_one(src, force, hdr_time):
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), hdr_time):
        return obj, None
    cmd = [HIPCC] + COMMON
    if src.endswith(".hip"):
        cmd += DEVICE
    else:
        cmd += ["-x", "c++"]        # host-only translation units: no device pass needed
    cmd += ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), log))
    return obj, log.strip() or None


def build(force=False, verbose=True):
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    hdr_time = headers_mtime()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(lambda s: compile_one(s, force, hdr_time), srcs))
    objs = [o for o, _ in results]
    for (_, log), src in zip(results, srcs):
        if log and verbose:
            print("[%s]\n%s" % (os.path.basename(src), log))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed: %s\n%s%s" % (" ".join(cmd), r.stdout, r.stderr))
    if verbose:
        print("built", LIB)
    return LIB


def build_c_caller(out=None, verbose=True):
    """Compile tests/c_caller.c, a host program in plain C against the public headers (the shape of the reference's
    own example program), with gcc and link it against the library.  Its _Static_assert block checks the struct
    layouts of include/dR_types.h against the reference's (tests/golden/ref_struct_offsets.h)."""
    tests = os.path.join(ROOT, "tests")
    out = out or os.path.join(tests, "bin", "c_caller")
    os.makedirs(os.path.dirname(out), exist_ok=True)
    cmd = [os.environ.get("CC", "gcc"), "-std=c11", "-O1", "-Wall", "-Werror", "-I" + os.path.join(ROOT, "include"), "-I" + tests,
           os.path.join(tests, "c_caller.c"), "-o", out, "-L" + LIBDIR, "-ldeepracin", "-Wl,-rpath," + LIBDIR,
           "-Wl,-rpath,$ORIGIN/../../deepracin_amd/lib"]       # (found from tests/bin wherever the tree is copied to)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s%s" % (" ".join(cmd), r.stdout, r.stderr))
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    build_c_caller()
