"""The build's report of kernels that use scratch memory.  A kernel that spills registers pays
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
