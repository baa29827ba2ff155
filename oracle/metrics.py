"""Parity metrics used by the tests (TEST INFRASTRUCTURE, see `oracle/__init__.py`)."""
import torch


def loss(out, ref, remove_zero=False):
  """Error summary in the form the reference prints (python/asuka/utils.py:61-76): elementwise
  abs/rel max and mean; integer tensors report the mismatch count."""
  assert out.shape == ref.shape, f"{out.shape=} {ref.shape=}"
  if out.dtype in (torch.int32, torch.int64):
    err_num = int((out != ref).sum())
    return {"err_num": err_num, "err": err_num / out.numel()}
  diff = (out.float() - ref.float()).abs()
  deno = ref.float().abs()
  if remove_zero:
    deno = torch.where(deno == 0, torch.ones_like(deno), deno)
  rel = diff / deno
  return {"abs_max": diff.max().item(), "abs_mean": diff.mean().item(),
          "rel_max": rel.max().item(), "rel_mean": rel.mean().item(), "remove_zero": remove_zero}


def rel_fro(out, ref):
  """Norm-wise relative error ||out-ref||_F / ||ref||_F."""
  return ((out.double() - ref.double()).norm() / ref.double().norm().clamp_min(1e-300)).item()


def topk_agreement(idx, ref_score, k, rtol=1e-3):
  """Heavy-hitter parity rule: per row of ref_score [..., S], the returned index set must contain every
  key whose reference score exceeds the k-th largest by more than the score tolerance, and may contain
  no key that falls short of it by more than the tolerance.  Returns the number of violating rows."""
  S = ref_score.shape[-1]
  flat_ref = ref_score.reshape(-1, S).double()
  flat_idx = idx.reshape(-1, idx.shape[-1]).long()
  bad = 0
  for r in range(flat_ref.shape[0]):
    row = flat_ref[r]
    kth = torch.topk(row, k).values[-1]
    tol = rtol * kth.abs()
    must = set(torch.nonzero(row > kth + tol).flatten().tolist())
    may = set(torch.nonzero(row >= kth - tol).flatten().tolist())
    got = set(flat_idx[r].tolist())
    if len(got) != k or not must.issubset(got) or not got.issubset(may):
      bad += 1
  return bad
