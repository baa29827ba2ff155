"""Harness helpers with the reference's interface (python/asuka/utils.py:28-76): `perf` times a callable
around device synchronisation and prints avg/min/max ms, `loss` reports abs/rel max/mean errors.

`perf(profile=True)` brackets the timed loop for a profiler as the reference does with cudaProfilerStart /
cudaProfilerStop (python/asuka/utils.py:15-25,35-36,45-46): here a roctx range named after the label plus
roctxProfilerResume / roctxProfilerPause, which `rocprofv3 --marker-trace` (and a collection started paused)
pick up.  Without the roctx library the bracket is a no-op."""
import ctypes
import threading
import time

import numpy as np
import torch

_roctx = None
_roctx_lock = threading.Lock()


def _load_roctx():
  global _roctx
  with _roctx_lock:
    if _roctx is None:
      _roctx = False
      for name in ("librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so"):
        try:
          lib = ctypes.CDLL(name)
          lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
          lib.roctxRangePushA.restype = ctypes.c_int
          lib.roctxRangePop.restype = ctypes.c_int
          _roctx = lib
          break
        except (OSError, AttributeError):
          continue
  return _roctx


def profile_start(label="perf"):
  """Open the profiled region: resume a paused collection and push a named range."""
  lib = _load_roctx()
  if lib:
    if hasattr(lib, "roctxProfilerResume"):
      lib.roctxProfilerResume(ctypes.c_uint64(0))
    lib.roctxRangePushA(str(label).encode())
  return bool(lib)


def profile_stop():
  """Close the region opened by profile_start."""
  lib = _load_roctx()
  if lib:
    lib.roctxRangePop()
    if hasattr(lib, "roctxProfilerPause"):
      lib.roctxProfilerPause(ctypes.c_uint64(0))
  return bool(lib)


def perf(label, f, args, kwargs={}, gflops=None, mem_gb=None, run=10, warmup=4, profile=False):
  torch.cuda.synchronize()
  for _ in range(warmup):
    f(*args, **kwargs)
    torch.cuda.synchronize()
  ms = []
  if profile:
    profile_start(label)
  for _ in range(run):
    torch.cuda.synchronize()
    tik = time.time()
    f(*args, **kwargs)
    torch.cuda.synchronize()
    ms.append((time.time() - tik) * 1000.0)
  if profile:
    profile_stop()
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
