"""What the compiler reported for the kernels of the hot path when the library was last built here
(macseek_amd/libmsq.kernels.json, written by macseek_amd.build): none of them may keep anything in scratch memory.

A kernel whose staging array or spilled registers land in scratch still passes every parity test and runs several
times slower (the small-N matvec did, at 17 us instead of 10, until its report was read), so the report is checked
like a result. Instantiations for rarely used shapes that are known to spill a few registers are not listed."""
import json
import os

import pytest

REPORT = os.path.join(os.path.dirname(__file__), "..", "macseek_amd", "libmsq.kernels.json")

# substrings of mangled names: every kernel whose name contains one of them must be free of scratch
NO_SCRATCH = [
    "13mv_tok_kernel",                                              # decode matvec and small-N matvec, every format
    "14mv_ring_kernel",
    "13moe_gu_kernelINS_8DecIQ1SQENS_10DecIQ2XXSQ",                   # BASELINE configs[2]
    "15moe_down_kernelINS_7DecIQ1SENS_9DecIQ2XXSELi768",
    "13moe_gu_kernelINS_10DecIQ2XXSQES1_",                            # IQ2_XXS routed + IQ2_XXS shared
    "19moe_pf_block_kernel",                                        # prefill grouped GEMM, BASELINE configs[3]
    "15mm_fused_kernel", "14mm_tile_kernel", "16mm_reduce_kernel",  # fused prefill matmul
    "19router_fused_kernel",
]


@pytest.fixture(scope="module")
def report():
    if not os.path.exists(REPORT):
        pytest.skip("no build report beside the library (built elsewhere)")
    with open(REPORT) as f:
        per_file = json.load(f)
    kernels = {}
    for ks in per_file.values():
        kernels.update(ks)
    return kernels


@pytest.mark.parametrize("pattern", NO_SCRATCH)
def test_hot_path_kernels_use_no_scratch(report, pattern):
    hits = {k: v for k, v in report.items() if pattern in k}
    assert hits, "no kernel matches %r: the list is out of date" % pattern
    bad = {k: v["scratch"] for k, v in hits.items() if v.get("scratch", 0) != 0}
    assert not bad, "kernels with scratch bytes per lane: %r" % bad


def test_report_covers_every_source(report):
    assert len(report) > 100  # the library holds a few hundred kernel instantiations
    for k, v in report.items():
        assert {"vgprs", "scratch", "lds"} <= set(v), k
