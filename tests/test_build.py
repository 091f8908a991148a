"""The build's checks of what the compiler made.  An MFMA that the compiler put under a mask of
lanes instead of a branch runs all the same (it does not look at the mask): the build lists the
device assembly and refuses such a kernel.  And the build's report of kernels that use scratch memory.  A kernel that spills registers pays
for more than its spills: a launch that needs scratch memory takes some 15 us longer, so the
library is kept free of such kernels and the build says so when one appears."""
import json
import os

from tffinfer_amd.kernels import build

REMARKS = """\
a.hip:10:1: remark: Function Name: _Z4goodPf [-Rpass-analysis=kernel-resource-usage]
a.hip:10:1: remark:     VGPRs: 24 [-Rpass-analysis=kernel-resource-usage]
a.hip:10:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:10:1: remark:     Occupancy [waves/SIMD]: 8 [-Rpass-analysis=kernel-resource-usage]
a.hip:20:1: remark: Function Name: _Z6spillsPf [-Rpass-analysis=kernel-resource-usage]
a.hip:20:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
a.hip:20:1: remark:     ScratchSize [bytes/lane]: 412 [-Rpass-analysis=kernel-resource-usage]
a.hip:30:1: warning: something else
"""


def test_scratch_users_are_read_from_the_remarks():
    assert build._scratch_users(REMARKS) == {"_Z6spillsPf": 412}
    assert build._scratch_users("") == {}


def test_the_built_library_has_no_kernel_with_scratch_memory():
    """Of the library in the tree, if there is one built from the present sources (the build
    writes what it found beside it)."""
    lib = build.find_library()
    if lib is None:
        import pytest
        pytest.skip("no library built from the present sources")
    with open(os.path.join(os.path.dirname(lib), "build_info.json")) as f:
        info = json.load(f)
    assert info.get("scratch_bytes_per_lane") == {}, info.get("scratch_bytes_per_lane")


LISTING = """\
_Z4goodv:                               ; @_Z4goodv
\ts_and_saveexec_b64 s[0:1], vcc
\ts_cbranch_execz .LBB0_2
\tv_mfma_f32_16x16x32_bf16 v[2:5], v[6:9], v[10:13], v[2:5]
.LBB0_2:
\ts_or_b64 exec, exec, s[0:1]
\ts_and_saveexec_b64 s[0:1], vcc
\tv_add_f32_e32 v1, v1, v2
\ts_or_b64 exec, exec, s[0:1]
\tv_mfma_f32_16x16x32_bf16 v[2:5], v[6:9], v[10:13], v[2:5]
\ts_endpgm
_Z3badv:                                ; @_Z3badv
\ts_and_saveexec_b64 s[2:3], vcc
\ts_waitcnt vmcnt(0)
\tv_mfma_f32_16x16x32_bf16 v[2:5], v[238:241], v[242:245], v[2:5]
\ts_or_b64 exec, exec, s[2:3]
\ts_and_saveexec_b64 s[2:3], vcc
\tv_mfma_f32_16x16x32_bf16 v[2:5], v[238:241], v[242:245], v[2:5]
\ts_or_b64 exec, exec, s[2:3]
\ts_endpgm
"""


def test_an_mfma_under_a_lane_mask_is_found_in_a_listing():
    assert build._masked_mfma(LISTING) == {"_Z3badv": 2}
    assert build._masked_mfma("") == {}


def test_the_built_library_has_no_mfma_under_a_lane_mask():
    """Of the library in the tree, if its build listed the assembly (every build does unless told not to)."""
    import pytest
    lib = build.find_library()
    if lib is None:
        pytest.skip("no library built from the present sources")
    with open(os.path.join(os.path.dirname(lib), "build_info.json")) as f:
        info = json.load(f)
    if "mfma_under_lane_mask" not in info:
        pytest.skip("the library was built without the check")
    assert info["mfma_under_lane_mask"] == {}
