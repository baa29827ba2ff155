"""The benchmarked kernels must not spill: a spilled register's reload is a scratch load, which waits in the same
counter (vmcnt) as the direct-to-LDS tile loads the loops keep in flight, so a single spill inside a loop
serialises the prefetch.  `flashtensor_amd.build` records the compiler's per-kernel resource usage next to each
object; this test reads those records (and is skipped when the library has not been built in this tree)."""
import json
import os

import pytest

from flashtensor_amd import build


def _load(src):
  path = build.resources_path(src)
  if not os.path.exists(path):
    pytest.skip(f"{os.path.basename(path)} not present: run python -m flashtensor_amd.build")
  with open(path) as f:
    return json.load(f)


def _one(res, fragment):
  hits = [(k, v) for k, v in res.items() if fragment in k]
  assert len(hits) == 1, (fragment, [k for k, _ in hits])
  return hits[0][1]


# attn_fwd_kernel<F16, 128, CAUSAL, EMU, KF, WAVES>: plain softmax in both forms, soft-cap and the packed
# KeyFormer mode of the large form
@pytest.mark.parametrize("fragment", [
    "attn_fwd_kernelINS_3F16ELi128ELb1ELb1ELi0ELi8E",
    "attn_fwd_kernelINS_3F16ELi128ELb1ELb1ELi0ELi4E",
    "attn_fwd_kernelINS_3F16ELi128ELb1ELb1ELi3ELi8E",
    "attn_fwd_kernelINS_3F16ELi128ELb1ELb1ELi4ELi8E",
])
def test_attention_kernels_of_the_benchmarked_configurations_do_not_spill(fragment):
  r = _one(_load("attn_fwd_f16_d128.hip"), fragment)
  assert r["vgpr_spill"] == 0 and r["scratch_bytes"] == 0, r  # (scalar registers spill to vector lanes, not to memory)
  assert r["vgprs"] + r["agprs"] <= 256 and r["occupancy"] == 2, r  # two waves per SIMD


# colstats_kernel<F16, 128, CAUSAL, EMU, MODE>: sum (H2O), sum of squares (RoCo), packed seeded KeyFormer (tau = 1 and
# general), CoRM rule: one score buffer reduced in place leaves registers for three waves per SIMD; the tensor-noise
# KeyFormer mode holds its prefetched slice instead and runs two
@pytest.mark.parametrize("mode,waves", [(0, 3), (1, 3), (6, 3), (7, 3), (4, 3), (2, 2)])
def test_column_pass_kernels_of_the_benchmarked_configurations_do_not_spill(mode, waves):
  r = _one(_load("colstats.hip"), f"colstats_kernelINS_3F16ELi128ELb1ELb1ELi{mode}E")
  assert r["vgpr_spill"] == 0 and r["scratch_bytes"] == 0, r
  assert r["occupancy"] >= waves, r


def test_linear_attention_kernels_do_not_spill():
  res = _load("linattn.hip")
  for name, r in res.items():
    if "linattn_" in name:
      assert r["vgpr_spill"] == 0 and r["scratch_bytes"] == 0, (name, r)
  # the two-launch block for narrow models: 8 waves per workgroup, so two per SIMD must fit
  res = _load("linblock_small.hip")
  assert len([n for n in res if "linblk_" in n]) == 30
  for name, r in res.items():
    if "linblk_" in name:
      assert r["vgpr_spill"] == 0 and r["scratch_bytes"] == 0 and r["occupancy"] >= 2, (name, r)
