"""The hot kernels are written for a fixed register budget: the 4-wave GEMM for one wave per SIMD with its
accumulators in AGPRs, the attention kernel for two waves per SIMD around a hand-placed assembly statement with
fixed registers.  A spill or a scratch access inside them is not only slow: the compiler's reloads are vector
memory operations that share the counter the kernels' own LDS-DMA requests are waited on with.  The build keeps
the compiler's per-kernel resource report beside each object; this test reads it."""
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REPORTS = os.path.join(ROOT, "graph-compiler_amd", "build", "kernels")


def _kernels():
    out = {}
    for path in glob.glob(os.path.join(REPORTS, "*.resources.txt")):
        cur = None
        for line in open(path, errors="replace"):
            m = re.search(r"remark:\s+Function Name: (\S+)", line)
            if m:
                cur = out.setdefault(m.group(1), {})
                continue
            m = re.search(r"remark:\s+([A-Za-z /\[\]]+?)(?: \[[^\]]*\])?: (\S+) \[-Rpass-analysis", line)
            if m and cur is not None:
                cur[m.group(1).strip()] = m.group(2)
    return out


@pytest.fixture(scope="module")
def kernels():
    k = _kernels()
    if not k:
        pytest.skip("no resource reports: the library has not been built in this tree")
    return k


def _pick(kernels, *parts):
    hits = {n: r for n, r in kernels.items() if all(p in n for p in parts)}
    assert hits, "no kernel whose name contains %s" % (parts,)
    return hits


@pytest.mark.parametrize("parts,occupancy,max_lds", [
    (("gemm_tile256_w4_kernel",), 1, 160 * 1024),      # one wave per SIMD: 256 AGPRs + the fragment sets
    (("mha_fwd_fast_kernel", "ELi4ELb1"), 2, 80 * 1024),  # pipelined attention: two workgroups per compute unit
    (("gemm_tile256_mi16_kernel",), 2, 160 * 1024),
    (("gemm_skinny_nt_kernel",), 2, 64 * 1024),
    (("gemm_rows32_kernel", "ILi2E"), 2, 72 * 1024),    # 8 waves and a ring of three 24 KiB stages: two per compute unit
    (("gemm_rows32_kernel", "ILi4E"), 2, 96 * 1024),    # 64 rows of A: three 32 KiB stages, one workgroup per compute unit
    (("gemm_rows32_kernel", "ILi8E"), 2, 144 * 1024),   # 128 rows of A: three 48 KiB stages
    (("gemm_tile128_kernel",), 2, 80 * 1024),           # small tiles: two workgroups per compute unit share its LDS
])
def test_hot_kernels_have_no_scratch_and_keep_their_occupancy(kernels, parts, occupancy, max_lds):
    for name, r in _pick(kernels, *parts).items():
        assert r.get("ScratchSize") == "0", (name, r)
        assert r.get("VGPRs Spill") == "0" and r.get("SGPRs Spill") == "0", (name, r)
        assert int(r["Occupancy"]) >= occupancy, (name, r)
        assert int(r["LDS Size"]) <= max_lds, (name, r)


def test_w4_gemm_keeps_its_accumulators_in_agprs(kernels):
    for name, r in _pick(kernels, "gemm_tile256_w4_kernel").items():
        assert int(r["AGPRs"]) == 256, (name, r)
