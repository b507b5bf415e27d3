"""Builds libedenhip.so (HIP kernels + the operator-level C ABI, include/eden_hip.h) for gfx950 with hipcc, and
libedenud.so (the C++ host classes behind the userdriver-level C ABI, include/eden_ud.h) with g++ against it.
Everything is built in-tree; nothing is installed."""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libedenhip.so")
UD_LIB = os.path.join(HERE, "libedenud.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


# MFMA results straight into ordinary registers for the kernels whose epilogue is the bottleneck (no AGPR -> VGPR
# copy per output); the big-tile GEMM keeps its accumulators in the AGPR half of the register file
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
PER_FILE_FLAGS = {"eh_gemm_thin.hip": VGPR_FORM, "eh_block.hip": VGPR_FORM, "eh_conv_c3.hip": VGPR_FORM, "eh_conv_rows.hip": VGPR_FORM}

RESOURCES = os.path.join(OBJ, "kernel_resources.txt")


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass of hipcc does not know the packed-fp32 feature and says so once per file: harmless
    lines = [l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l]
    remarks, rest, after_remark = [], [], False
    for l in lines:
        if "-Rpass-analysis=kernel-resource-usage" in l:
            remarks.append(l)
            after_remark = True
        elif after_remark and re.match(r"^\s*(\d+\s*)?\|", l):
            pass  # the source line and caret the compiler prints under a remark
        else:
            rest.append(l)
            after_remark = False
    out = "\n".join(rest)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)
    return remarks


def _resource_table(remarks):
    """'kernel vgprs agprs scratch_bytes_per_lane waves_per_simd' lines from the compiler's resource remarks"""
    rows, cur = [], None
    for l in remarks:
        m = re.search(r"Function Name: (\S+)", l)
        if m:
            cur = {"name": m.group(1)}
            rows.append(cur)
            continue
        for key, pat in (("vgprs", r" VGPRs: (\d+)"), ("agprs", r"AGPRs: (\d+)"), ("scratch", r"ScratchSize \[bytes/lane\]: (\d+)"),
                         ("occupancy", r"Occupancy \[waves/SIMD\]: (\d+)")):
            m = re.search(pat, l)
            if m and cur is not None:
                cur[key] = int(m.group(1))
    return ["%s %d %d %d %d" % (r["name"], r.get("vgprs", -1), r.get("agprs", -1), r.get("scratch", -1), r.get("occupancy", -1))
            for r in rows]


def build_lib(jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    objs = [os.path.join(OBJ, f[:-4] + ".o") for f in srcs]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        remarks = list(ex.map(lambda so: _run([HIPCC, *HIP_FLAGS, *PER_FILE_FLAGS.get(so[0], []),
                                               "-Rpass-analysis=kernel-resource-usage", "-c",
                                               os.path.join(CSRC, so[0]), "-o", so[1]]), zip(srcs, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    # registers, spill bytes and occupancy of every kernel, for the test that guards the hot kernels' budgets
    with open(RESOURCES, "w") as f:
        for src, r in zip(srcs, remarks):
            for row in _resource_table(r):
                f.write(src + " " + row + "\n")
    return LIB


def build_ud_lib():
    """The userdriver level: host/*.hpp (header-only C++ classes) behind host/ud_c_api.cpp, linked against libedenhip.so."""
    _run(["g++", "-O2", "-std=c++17", "-Wall", "-fPIC", "-shared", "-I" + os.path.join(ROOT, "include"), "-I" + HOST,
          os.path.join(HOST, "ud_c_api.cpp"), "-o", UD_LIB, "-L" + HERE, "-ledenhip", "-Wl,-rpath,$ORIGIN"])
    return UD_LIB


def build_all():
    lib = build_lib()
    build_ud_lib()
    return lib


if __name__ == "__main__":
    print(build_all())
    sys.exit(0)
