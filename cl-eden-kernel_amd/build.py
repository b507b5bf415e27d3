"""Builds libedenhip.so (HIP kernels + C ABI) and libedenhip_ud.so's test driver
for gfx950 with hipcc.  Everything is built in-tree; nothing is installed."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libedenhip.so")
UD_TEST = os.path.join(HERE, "ud_op_test")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass of hipcc does not know the packed-fp32 feature and says so once per file: harmless
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build_lib(jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    objs = [os.path.join(OBJ, f[:-4] + ".o") for f in srcs]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _run([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, so[0]), "-o", so[1]]), zip(srcs, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


def build_ud_test():
    """The C++ operator classes (header-only, host/) with their test driver, linked against libedenhip.so."""
    src = os.path.join(HOST, "ud_op_test.cpp")
    if not os.path.exists(src):
        return None
    _run(["g++", "-O2", "-std=c++17", "-Wall", "-I" + os.path.join(ROOT, "include"), "-I" + HOST,
          "-I" + os.path.join(ROOT, "oracle"), src, "-o", UD_TEST,
          "-L" + HERE, "-ledenhip", "-Wl,-rpath,$ORIGIN", "-L" + os.path.join(ROOT, "oracle"), "-loracle",
          "-Wl,-rpath,$ORIGIN/../oracle"])
    return UD_TEST


def build_all():
    lib = build_lib()
    build_ud_test()
    return lib


if __name__ == "__main__":
    print(build_all())
    sys.exit(0)
