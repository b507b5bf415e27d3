"""Builds the C++ test driver of the operator classes (tests/ud_op_test.cpp): the header-only host classes of the
package compiled together with the tests and linked against libedenhip.so and the CPU oracle.  The oracle is linked
into this test program only; nothing in the package includes or links it."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
PKG = os.path.join(ROOT, "cl-eden-kernel_amd")
BIN = os.path.join(HERE, "ud_op_test")


def build_ud_test():
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(PKG, "host"),
           "-I" + os.path.join(ROOT, "oracle"), os.path.join(HERE, "ud_op_test.cpp"), "-o", BIN,
           "-L" + PKG, "-ledenhip", "-Wl,-rpath,$ORIGIN/../cl-eden-kernel_amd", "-L" + os.path.join(ROOT, "oracle"), "-loracle",
           "-Wl,-rpath,$ORIGIN/../oracle", "-pthread"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), r.stdout))
    if r.stdout.strip():
        print(r.stdout)
    return BIN


if __name__ == "__main__":
    print(build_ud_test())
