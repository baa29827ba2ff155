"""Harness helpers with the reference's interface (python/asuka/utils.py:28-76): `perf` times a callable
around device synchronisation and prints avg/min/max ms, `loss` reports abs/rel max/mean errors."""
import time

import numpy as np
import torch


def perf(label, f, args, kwargs={}, gflops=None, mem_gb=None, run=10, warmup=4, profile=False):
  torch.cuda.synchronize()
  for _ in range(warmup):
    f(*args, **kwargs)
    torch.cuda.synchronize()
  ms = []
  for _ in range(run):
    torch.cuda.synchronize()
    tik = time.time()
    f(*args, **kwargs)
    torch.cuda.synchronize()
    ms.append((time.time() - tik) * 1000.0)
  avg_ms, min_ms, max_ms = float(np.mean(ms)), float(np.min(ms)), float(np.max(ms))
  msg = f"[{label}] avg {avg_ms:.4f} ms, min {min_ms:.4f} ms, max {max_ms:.4f} ms"
  if gflops is not None:
    msg += f", {gflops / (avg_ms / 1000.0)} gflops/s"
  if mem_gb is not None:
    msg += f", {mem_gb / (avg_ms / 1000.0)} gb/s"
  msg += f" ({run} runs, {warmup} warmups" + (", profiled)" if profile else ")")
  print(msg)
  return avg_ms


def loss(out, ref, remove_zero=False):
  assert out.shape == ref.shape, f"{out.shape=} {ref.shape=}"
  if out.dtype in {torch.int32, torch.int64}:
    err_num = torch.sum(out != ref).item()
    return {"err_num": err_num, "err": err_num / out.numel()}
  diff = (out.float() - ref.float()).abs()
  deno = ref.float().abs()
  if remove_zero:
    deno = torch.where(deno == 0, torch.ones_like(deno), deno)
  rel = diff / deno
  return {"abs_max": diff.max().item(), "abs_mean": diff.mean().item(), "rel_max": rel.max().item(),
          "rel_mean": rel.mean().item(), "remove_zero": remove_zero}
