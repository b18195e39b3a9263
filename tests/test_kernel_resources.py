"""Register and scratch use of the kernels that count their own vector-memory operations (CPU: hipcc compiles the
source to assembly for gfx950, nothing runs).

The sparse attention kernels issue their tile copies through inline asm and wait for them with
`s_waitcnt vmcnt(n)`, n being the number of operations issued since. A register spilled to scratch adds a
vector-memory operation that nobody counted, and its reload waits for every copy in flight. Zero scratch is
therefore part of these kernels' contract, not a tuning detail.

The second rule checked here: no inline asm statement loads into a register. The compiler takes an asm output for
valid as soon as the statement ends and may move, reuse or spill that register while the load is in flight; only
loads whose destination is LDS (they write no register) are issued through asm, every other load is an ordinary
one that the compiler waits for itself.
"""
import os
import shutil

import pytest

from moespresso_amd import build

pytestmark = pytest.mark.skipif(not (os.path.exists(build.HIPCC) or shutil.which(build.HIPCC)), reason="hipcc not installed")


@pytest.fixture(scope="module")
def sparse_assembly():
    return build.device_assembly(os.path.join(build.CSRC, "sparse_attn.hip"))


@pytest.fixture(scope="module")
def sparse_kernels(sparse_assembly):
    return build.kernel_resources(os.path.join(build.CSRC, "sparse_attn.hip"), sparse_assembly)


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


def test_no_inline_asm_statement_loads_into_a_register(sparse_assembly):
    bodies = build.kernel_bodies(sparse_assembly)
    assert any("sparse_attn_prefill_kernel" in k for k in bodies) and len(bodies) >= 11, sorted(bodies)
    for name, lines in bodies.items():
        assert build.inline_asm_register_loads(lines) == [], name
    # the rule has teeth: the same scan flags a register load inside an asm block
    sample = ["\t;;#ASMSTART", "\tglobal_load_dword v3, v[4:5], off", "\t;;#ASMEND",
              "\t;;#ASMSTART", "\tglobal_load_lds_dwordx4 v[4:5], off", "\t;;#ASMEND", "\tglobal_load_dword v9, v[4:5], off"]
    assert build.inline_asm_register_loads(sample) == ["global_load_dword v3, v[4:5], off"]


def test_prefill_consumer_store_count_matches_what_its_waits_assume(sparse_assembly):
    """The persistent prefill consumer counts sixteen output stores per unit and wave into its wait counts (a count
    above what was issued would end a wait early); the compiler must issue exactly that many, and no other store."""
    (name, lines), = [(k, v) for k, v in build.kernel_bodies(sparse_assembly).items() if "sparse_attn_prefill_kernel" in k]
    stores = [l.split()[0] for l in lines if l.strip().startswith(("global_store", "flat_store", "buffer_store", "scratch_store"))]
    assert stores == ["global_store_dwordx4"] * 16, stores
    # compiler-visible loads: the sixteen query loads at each of their two places, the sink (two forms, two places)
    loads = [l.split()[0] for l in lines if l.strip().startswith(("global_load", "flat_load", "buffer_load", "scratch_load"))
             and "_lds_" not in l]
    assert loads.count("global_load_dwordx4") == 32 and len(loads) == 36, loads
