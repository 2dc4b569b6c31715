"""What the compiler reported for every HIP kernel of the last build (paralia-framework_amd/build/**/*.hip.o.log, written by
the Makefile with -Rpass-analysis=kernel-resource-usage): no kernel may spill registers to scratch memory (a spilling
tile kernel computes the right numbers thirty times slower; the Makefile refuses to link one, this test says which),
and the tile kernels must keep the occupancy their design counts on."""
import glob
import os
import re

import pytest

BUILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "paralia-framework_amd", "build")


def kernels():
    out = {}
    for path in glob.glob(os.path.join(BUILD, "**", "*.hip.o.log"), recursive=True):
        name = None
        for line in open(path, errors="replace"):
            m = re.search(r"remark: Function Name: (\S+)", line)
            if m:
                name = m.group(1)
                out[name] = {"file": os.path.basename(path)}
                continue
            m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\S+) \[-Rpass-analysis", line)
            if m and name:
                out[name][m.group(1).strip()] = m.group(2)
    return out


def test_no_kernel_spills_and_tile_kernels_keep_their_occupancy():
    ks = kernels()
    if not ks:
        pytest.skip("no build logs: run make -C paralia-framework_amd (or __graft_entry__.build()) first")
    gemm = {n: k for n, k in ks.items() if "gemm_kernel" in n}
    assert len(gemm) >= 20, sorted(ks)             # fp64 x 4 transposes x 2, fp32 small / wide / large
    for n, k in ks.items():
        assert k["ScratchSize"] == "0" and k["VGPRs Spill"] == "0" and k["SGPRs Spill"] == "0", (n, k)
    for n, k in gemm.items():
        large = "Li256ELi256E" in n
        # the 256 x 256 fp32 tile holds a compute unit alone (256 accumulator registers in AGPRs, 144 KiB of LDS);
        # every other tile must leave room for a second workgroup per compute unit: at most 256 registers per lane
        assert int(k["Occupancy"]) >= (1 if large else 2), (n, k)
        if large:
            assert int(k["AGPRs"]) == 256 and int(k["LDS Size"]) <= 160 * 1024, (n, k)
        else:
            assert int(k["LDS Size"]) <= 80 * 1024, (n, k)
