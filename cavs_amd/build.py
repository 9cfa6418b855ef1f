"""Builds the HIP backend (libcavs_hip.so) and the host runtime (libcavs_host.so)
in-tree with hipcc / g++ for gfx950.  Run as `python -m cavs_amd.build`."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(PKG, "build")
HIP_SO = os.path.join(LIB, "libcavs_hip.so")
HOST_SO = os.path.join(LIB, "libcavs_host.so")
APPS_SO = os.path.join(LIB, "libcavs_apps.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-I", os.path.join(ROOT, "include"),
             "-I", CSRC, "-Wall", "-Wno-unused-function",
             # packed fp32 math is disabled on this target by policy
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
CXX = os.environ.get("CXX", "g++")
CXX_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-missing-field-initializers", "-I",
             os.path.join(ROOT, "include"), "-I", HOST]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + r.stderr)
        raise RuntimeError("build step failed: " + os.path.basename(cmd[-1]))
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")


def build_hip(jobs=8):
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _run([HIPCC] + HIP_FLAGS + ["-c", so[0], "-o", so[1]]), zip(srcs, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_SO] + objs + ["-lhiprtc"])
    return HIP_SO


def build_host():
    srcs = sorted(glob.glob(os.path.join(HOST, "*.cc")) + glob.glob(os.path.join(HOST, "frontend", "*.cc")) +
                  glob.glob(os.path.join(HOST, "midend", "*.cc")))
    if not srcs:
        return None
    os.makedirs(OBJ, exist_ok=True)
    objs = [os.path.join(OBJ, "host_" + os.path.relpath(s, HOST).replace(os.sep, "_")[:-3] + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=8) as ex:
        list(ex.map(lambda so: _run([CXX] + CXX_FLAGS + ["-c", so[0], "-o", so[1]]), zip(srcs, objs)))
    _run([CXX, "-shared", "-o", HOST_SO] + objs + ["-L", LIB, "-lcavs_hip", "-Wl,-rpath,$ORIGIN"])
    # the benchmark applications written against the front end (a user-side program)
    apps = sorted(glob.glob(os.path.join(HOST, "apps", "*.cc")))
    if apps:
        _run([CXX] + CXX_FLAGS + ["-shared", "-o", APPS_SO] + apps +
             ["-L", LIB, "-lcavs_host", "-lcavs_hip", "-Wl,-rpath,$ORIGIN"])
    return HOST_SO


def build_all():
    return build_hip(), build_host()


if __name__ == "__main__":
    print(build_all())
