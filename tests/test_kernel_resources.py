"""Register and spill budgets of the hot kernels, read from the table the build writes
(cl-eden-kernel_amd/build/kernel_resources.txt: file, kernel, VGPRs, AGPRs, scratch bytes per lane,
waves per SIMD).  A change that makes the compiler spill inside a GEMM tile costs a multiple of the
kernel's time and no parity test notices it, so the budgets are checked here, on the CPU."""
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TABLE = os.path.join(ROOT, "cl-eden-kernel_amd", "build", "kernel_resources.txt")


def rows():
    if not os.path.exists(TABLE):
        import importlib
        importlib.import_module("cl-eden-kernel_amd.build").build_lib()
    out = []
    for line in open(TABLE):
        f, name, vgprs, agprs, scratch, occ = line.split()
        out.append((f, name, int(vgprs), int(agprs), int(scratch), int(occ)))
    return out


def test_every_kernel_is_listed():
    names = [r[1] for r in rows()]
    for needle in ("igemm_dma_kernel", "direct_gemm_kernel", "conv_c3k3_kernel", "igemm_u8_kernel", "dw3x3_nhwc_tile4_kernel",
                   "add_u8_kernel", "avgpool_nhwc_vec4_kernel"):
        assert any(needle in n for n in names), needle


def test_tiled_gemm_kernels_do_not_spill():
    """The 256 x 256 tile holds 256 accumulator registers and every other register of the wave; a few
    bytes of scratch outside the loop are tolerated, the kilobyte a careless epilogue costs is not."""
    seen = 0
    for f, name, vgprs, agprs, scratch, occ in rows():
        if "igemm_dma_kernel" in name:
            seen += 1
            assert scratch <= 16, (name, scratch)
    assert seen == 28


@pytest.mark.parametrize("needle,max_scratch,min_occupancy", [
    ("direct_gemm_kernel", 0, 2),
    ("conv_c3k3_kernel", 0, 8),
    ("igemm_u8_kernel", 0, 3),
    ("dw3x3_nhwc_tile4_kernel", 0, 6),
    ("dw_nhwc_vec4_kernel", 0, 8),
    ("add_u8_kernel", 0, 8),
    ("avgpool_nhwc_vec4_kernel", 0, 8),
])
def test_other_hot_kernels_keep_their_occupancy(needle, max_scratch, min_occupancy):
    hits = [r for r in rows() if needle in r[1]]
    assert hits
    for f, name, vgprs, agprs, scratch, occ in hits:
        assert scratch <= max_scratch and occ >= min_occupancy, (name, scratch, occ)
