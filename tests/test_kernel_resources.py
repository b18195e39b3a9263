"""Register and scratch use of the kernels that count their own vector-memory operations (CPU: hipcc compiles the
source to assembly for gfx950, nothing runs).

The sparse attention kernels issue their tile copies through inline asm and wait for them with
`s_waitcnt vmcnt(n)`, n being the number of operations issued since. A register spilled to scratch adds a
vector-memory operation that nobody counted, and its reload waits for every copy in flight; the persistent prefill
consumer also relies on its query and id registers staying where the loads put them. Zero scratch is therefore part
of these kernels' contract, not a tuning detail.
"""
import os
import shutil

import pytest

from moespresso_amd import build

pytestmark = pytest.mark.skipif(not (os.path.exists(build.HIPCC) or shutil.which(build.HIPCC)), reason="hipcc not installed")


@pytest.fixture(scope="module")
def sparse_kernels():
    return build.kernel_resources(os.path.join(build.CSRC, "sparse_attn.hip"))


def test_sparse_attention_kernels_use_no_scratch(sparse_kernels):
    counted = {k: v for k, v in sparse_kernels.items() if "sparse_attn_split_kernel" in k or "sparse_attn_prefill_kernel" in k}
    # six instances of the split kernel (element type x row width x query type x rope) and the prefill consumer
    assert len(counted) == 7, sorted(counted)
    for name, res in counted.items():
        assert res["scratch_bytes"] == 0 and res["vgpr_spills"] == 0, (name, res)
        # eight waves per workgroup, one workgroup per CU: 256 registers per lane are there, not one more
        assert res["vgprs"] <= 256, (name, res)


def test_resource_query_sees_every_kernel_of_the_source(sparse_kernels):
    assert sum("sparse_attn_merge_kernel" in k for k in sparse_kernels) == 3
    for res in sparse_kernels.values():
        assert set(res) == {"vgprs", "sgprs", "scratch_bytes", "vgpr_spills", "sgpr_spills"} and res["vgprs"] > 0
