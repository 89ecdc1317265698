"""The register budget of the first-pass search kernels, checked on the compiler's own output (no GPU needed).

The sorted-set search is held to a fixed number of wavefronts per SIMD and runs 7 to 12 % slower when the register
allocator reloads a spilled register inside its hop loop; small source changes anywhere in the kernel decide that.
So every change is checked here: wavefronts per SIMD, scratch bytes per lane, and scratch-memory instructions inside
the hop loops (the innermost loops that hold both the sorted-set insert and a fetch from global memory)."""
import shutil

import pytest

from cuhnsw_amd import kernel_report

pytestmark = pytest.mark.skipif(shutil.which(kernel_report.HIPCC) is None, reason="hipcc is not installed")

# kernel -> (wavefronts per SIMD at least, scratch bytes per lane at most)
LIMITS = {
    "search_fast_kernel<dot,1,5>": (7, 68),
    "search_fast_kernel<dot,1,5,trails>": (7, 56),
    "search_fast_kernel<l2,1,5>": (7, 60),
    "search_fast_kernel<dot,2,5>": (7, 60),
    "search_fast_kernel<l2,2,5>": (7, 88),
    "search_fast_kernel<l2,2,5,trails>": (7, 76),
    "search_fast_kernel<dot,1,2>": (7, 0),
    "search_fast_kernel<dot,2,8>": (5, 36),
}


@pytest.fixture(scope="module")
def report():
  return kernel_report.compile_kernels(kernel_report.FIRST_PASS)


@pytest.mark.parametrize("name", sorted(LIMITS))
def test_first_pass_kernel_keeps_its_register_budget(report, name):
  waves, scratch = LIMITS[name]
  r = report[name]
  assert r["waves_per_simd"] >= waves, r
  assert r["scratch_bytes_per_lane"] <= scratch, r
  assert r["scratch_instructions_in_hop_loops"] == 0, r


def test_loop_analysis_sees_a_spill_inside_a_loop():
  """The control-flow analysis itself, on a hand-written listing: a query loop around a hop loop that holds a
  fetch and the insert; the scratch access in the hop loop counts, the ones outside it do not."""
  isa = """
kern:
  s_mov_b32 s0, 0
.LBB0_1:
  scratch_load_dword v1, off, off
  s_cbranch_scc1 .LBB0_5
.LBB0_2:
  global_load_dword v5, v[6:7], off
  v_med3_f32 v0, v1, v2, v3
  s_cbranch_vccz .LBB0_4
.LBB0_3:
  scratch_load_dword v2, off, off offset:4
.LBB0_4:
  s_cbranch_scc0 .LBB0_2
.LBB0_5:
  scratch_store_dword off, v1, off
  s_cbranch_scc0 .LBB0_1
.LBB0_6:
  s_endpgm
.Lfunc_end0:
"""
  assert kernel_report.loop_scratch_accesses(isa, "kern") == (1, 3)
