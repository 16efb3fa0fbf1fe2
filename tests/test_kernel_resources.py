"""Build-time check of the MFMA kernels' register budgets (CPU only: hipcc cross-compiles, nothing runs).

The kernels that walk tiles count their own s_waitcnt vmcnt around direct-to-LDS loads.  A register spilled to scratch
memory inside such a walk is reloaded with a vector memory load, which the hand-counted waits then cover too (the
epilogue ends up waiting for the next tile's prefetch), and a change of occupancy means that the compiler no longer gives a
wave the whole register file.  Both come and go with small source changes and with the compiler version, so the table
the compiler reports is held to its class here: profiles/kernel_resources.txt is the table this was last checked
against."""
import shutil

import pytest

from slowrun_amd import build

pytestmark = pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")

# one wave per SIMD, all accumulators in registers, nothing in scratch memory
HOT = ["fwd_kernel<true, false, true>", "fwd_kernel<true, false, false>", "fwd_kernel<false, false, true>", "fwd_kernel<false, false, false>",
       "fwd_kernel<false, true, false>", "fwd_sample_kernel<true, true>", "fwd_sample_kernel<false, true>", "bwd_recompute_kernel",
       "bwd_dx_kernel<bf16_t, false>", "bwd_dx_kernel<float, false>", "bwd_dx_kernel<bf16_t, true>", "bwd_dx_kernel<float, true>",
       "bwd_dw_kernel<false>", "bwd_dw_kernel<true>", "bwd_dw_tail_kernel", "bench_gemm_kernel", "floor_fwd_kernel", "floor_dx_kernel",
       "floor_dw_kernel"]
# the same, except that the compiler keeps part of the accumulators in architectural registers (its epilogue is a few stores)
HOT_ANY_AGPRS = ["fwd_sample_kernel<true, false>"]
# known to spill to scratch (a measurement aid); the bound is what was measured, so that it does not grow unseen
SCRATCH_BOUND = {"bench_mfma_kernel": 16}


@pytest.fixture(scope="module")
def table():
    return build.kernel_resources()


def test_every_kernel_is_reported(table):
    for k in HOT + HOT_ANY_AGPRS + list(SCRATCH_BOUND):
        assert k in table, f"{k} missing from the compiler's resource remarks: {sorted(table)}"


@pytest.mark.parametrize("kernel", HOT)
def test_hot_mfma_kernels_keep_everything_in_registers(table, kernel):
    r = table[kernel]
    assert r["scratch"] == 0 and r["vgpr_spill"] == 0, f"{kernel} spills to scratch memory: {r}"
    assert r["occupancy"] == 1 and r["agprs"] == 256, f"{kernel}: one wave per SIMD with 256 accumulation registers expected: {r}"


@pytest.mark.parametrize("kernel", HOT_ANY_AGPRS)
def test_other_mfma_kernels_keep_everything_in_registers(table, kernel):
    r = table[kernel]
    assert r["scratch"] == 0 and r["vgpr_spill"] == 0 and r["occupancy"] == 1, f"{kernel}: {r}"


@pytest.mark.parametrize("kernel", sorted(SCRATCH_BOUND))
def test_known_scratch_users_do_not_grow(table, kernel):
    r = table[kernel]
    assert r["scratch"] <= SCRATCH_BOUND[kernel], f"{kernel}: {r}"
    assert r["occupancy"] == 1


def test_no_other_kernel_uses_scratch(table):
    bad = {k: r["scratch"] for k, r in table.items() if r["scratch"] > 0 and k not in SCRATCH_BOUND}
    assert not bad, bad


def test_toolchain_is_recorded():
    v = build.hipcc_version()
    assert v, "hipcc --version gives no HIP version line"
    # not a failure when it differs (the build prints a warning): the table above is the check that matters
    print("hipcc HIP version", v, "tested with", build.TESTED_HIPCC)
