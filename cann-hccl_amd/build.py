"""Builds libhccl.so (the HIP library behind include/hccl/hccl.h) for gfx950 with hipcc.

    python cann-hccl_amd/build.py [--force]

Objects go to cann-hccl_amd/build/, the library to cann-hccl_amd/lib/libhccl.so.  The thirteen
kernel translation units (one per element type plus the byte-copy variants) compile in parallel.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libhccl.so")
ABI_CALLER = os.path.join(LIBDIR, "abi_caller")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-I", os.path.join(ROOT, "include"), "-I", CSRC,
          "-Wall", "-Wno-unused-command-line-argument"]
# gfx950 only; packed fp32 instructions are switched off for device code
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
DTYPES = list(range(12)) + [255]
DEVICE_SOURCES = ["noalloc.hip"]
HOST_SOURCES = ["plan.cc", "plan_schedules.cc", "plan_lower.cc", "plan_fuse.cc", "plan_template.cc", "ranktable.cc", "exec.cc", "api.cc", "api_rendezvous.cc", "api_comm.cc", "api_ext.cc", "kernels_table.cc"]


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(force=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers += [os.path.join(ROOT, "include", "hccl", f) for f in os.listdir(os.path.join(ROOT, "include", "hccl"))]
    jobs = jobs or min(8, os.cpu_count() or 4)
    tasks, objs = [], []
    for dt in DTYPES:
        obj = os.path.join(OBJ, "kernels_dt%d.o" % dt)
        objs.append(obj)
        src = os.path.join(CSRC, "kernels_dt.hip")
        if force or _newer(obj, [src] + headers):
            tasks.append([HIPCC] + COMMON + DEVICE + ["-DHCCL_DT=%d" % dt, "-c", src, "-o", obj])
    for name in DEVICE_SOURCES:
        obj = os.path.join(OBJ, name.replace(".hip", ".o"))
        objs.append(obj)
        src = os.path.join(CSRC, name)
        if force or _newer(obj, [src] + headers):
            tasks.append([HIPCC] + COMMON + DEVICE + ["-c", src, "-o", obj])
    for name in HOST_SOURCES:
        obj = os.path.join(OBJ, name.replace(".cc", ".o"))
        objs.append(obj)
        src = os.path.join(CSRC, name)
        if force or _newer(obj, [src] + headers):
            tasks.append([HIPCC] + COMMON + ["-D__HIP_PLATFORM_AMD__", "-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for out in ex.map(_run, tasks):
            if out:
                sys.stderr.write(out + "\n")
    if force or tasks or _newer(LIB, objs):
        _run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs + ["-lpthread"])
    build_abi_caller(force)
    build_threads_latency(force)
    return LIB


def build_abi_caller(force=False, include_dirs=None, out=None):
    """Links the C-ABI conformance program (tests/c_abi/caller.cc) against the library.  include_dirs
    lets a test put another header tree in front of this repository's include/."""
    src = os.path.join(ROOT, "tests", "c_abi", "caller.cc")
    out = out or ABI_CALLER
    if not os.path.exists(src):
        return None
    if force or include_dirs or _newer(out, [src, LIB]):
        inc = []
        for d in (include_dirs or []) + [os.path.join(ROOT, "include")]:
            inc += ["-I", d]
        _run([HIPCC, "-O1", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-Wno-unused-command-line-argument"] + inc +
             [src, "-L", LIBDIR, "-lhccl", "-Wl,-rpath,$ORIGIN", "-o", out])
    return out


def build_threads_latency(force=False):
    """Links the calling-model timing program (tests/c_abi/threads_latency.cc) against the library."""
    src = os.path.join(ROOT, "tests", "c_abi", "threads_latency.cc")
    out = os.path.join(LIBDIR, "threads_latency")
    if not os.path.exists(src):
        return None
    if force or _newer(out, [src, LIB]):
        _run([HIPCC, "-O2", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"),
              src, "-L", LIBDIR, "-lhccl", "-lpthread", "-Wl,-rpath,$ORIGIN", "-o", out])
    return out


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
