"""ft_attn_colstats_fwd_static, the entry point that allocates nothing (its scratch is a static device buffer of
the library), against ft_attn_colstats_fwd on the same inputs, through the C ABI: two calls in a row, the second
on a smaller problem (the buffer keeps the first call's contents), then grouped queries, the size limit and the
argument checks."""
import ctypes

import pytest
import torch

import oracle
from flashtensor_amd import _lib
from flashtensor_amd._lib import FtAttnArgs, FtStrides

pytestmark = pytest.mark.gpu


def _strides(t):
  return FtStrides(t.stride(0), t.stride(1), t.stride(2))


def _call_both(lib, gpu, B, S, H, D, seed, want_sq, Hkv=None, Skv=None):
  q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed, kv_len=Skv)
  if Hkv:
    k, v = k[:, :, :Hkv].contiguous(), v[:, :, :Hkv].contiguous()
  qd, kd, vd = q.to(gpu), k.to(gpu), v.to(gpu)
  Skv, Hs = kd.shape[1], kd.shape[2]
  stream = ctypes.c_void_p(torch.cuda.current_stream(gpu).cuda_stream)
  res = []
  for static in (False, True):
    out = torch.full_like(qd, float("nan"))
    s1 = torch.full((B, Hs, Skv), float("nan"), dtype=torch.float32, device=gpu)
    s2 = torch.full((B, H, Skv), float("nan"), dtype=torch.float32, device=gpu) if want_sq else None
    a = FtAttnArgs(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), _strides(qd), _strides(kd), _strides(vd),
                   _strides(out), B, H, S, Skv, D, _lib.FT_F16, _lib.FT_CAUSAL, Hs)
    if static:
      rc = lib.ft_attn_colstats_fwd_static(ctypes.byref(a), s1.data_ptr(), s2.data_ptr() if want_sq else None, stream)
    else:
      nbytes = lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(a))
      ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
      rc = lib.ft_attn_colstats_fwd(ctypes.byref(a), s1.data_ptr(), s2.data_ptr() if want_sq else None, ws.data_ptr(), nbytes, stream)
    assert rc == _lib.FT_OK, lib.ft_last_error().decode()
    torch.cuda.synchronize()
    res.append((out, s1, s2))
  return (q, k, v), res


def test_static_scratch_entry_point_matches_the_workspace_one(gpu):
  lib = _lib.load()
  # two calls in a row on the same GPU; the second, smaller problem finds the first one's normalisers in the buffer
  for (B, S, H, D, seed, want_sq) in [(2, 1000, 4, 128, 11, True), (1, 300, 2, 64, 12, False), (1, 130, 2, 128, 13, True)]:
    (q, k, v), (ref, got) = _call_both(lib, gpu, B, S, H, D, seed, want_sq)
    for r, g in zip(ref, got):
      if r is not None:
        assert torch.isfinite(g).all() and torch.equal(r, g)      # same kernels, same arithmetic: bit for bit
    # and both agree with the CPU definition
    ro, r1, r2 = oracle.roco_forward(q, k, v)
    assert (got[0].float().cpu() - ro.float()).abs().max().item() <= 2e-2
    assert ((got[1].cpu() - r1).abs() / r1).max().item() <= 1e-3 + 4e-3 / 1
  # grouped queries use the second part of the scratch (per-head sums before the group mean); rectangular problem
  (q, k, v), (ref, got) = _call_both(lib, gpu, 1, 200, 8, 128, 14, False, Hkv=2, Skv=264)
  assert torch.equal(ref[0], got[0]) and torch.equal(ref[1], got[1]) and got[1].shape == (1, 2, 264)


def test_static_scratch_entry_point_at_the_benchmarked_shape_and_under_graph_capture(gpu):
  """B1 H32 S4096 D128 (512 KB of normalisers, the 256-row two-block launch) bit for bit against the workspace entry
  point; then the same call recorded into a HIP graph (after the eager call above has looked the buffer up) and
  replayed on new inputs, with eager work between the replays."""
  lib = _lib.load()
  (q, k, v), (ref, got) = _call_both(lib, gpu, 1, 4096, 32, 128, 0, True)
  for r, g in zip(ref, got):
    assert torch.isfinite(g).all() and torch.equal(r, g)
  assert torch.allclose(got[1].sum(-1).cpu(), torch.full((1, 32), 4096.0), rtol=1e-4)
  B, S, H, D = 1, 600, 4, 128
  qd, kd, vd = (torch.zeros(B, S, H, D, dtype=torch.float16, device=gpu) for _ in range(3))
  out = torch.empty_like(qd)
  s1 = torch.empty(B, H, S, dtype=torch.float32, device=gpu)
  a = FtAttnArgs(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), _strides(qd), _strides(kd), _strides(vd),
                 _strides(out), B, H, S, S, D, _lib.FT_F16, _lib.FT_CAUSAL, H)
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    stream = ctypes.c_void_p(torch.cuda.current_stream(gpu).cuda_stream)
    assert lib.ft_attn_colstats_fwd_static(ctypes.byref(a), s1.data_ptr(), None, stream) == _lib.FT_OK, lib.ft_last_error().decode()
  for seed in (41, 42, 43):
    q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
    for dst, src in zip((qd, kd, vd), (q, k, v)):
      dst.copy_(src.to(gpu))
    graph.replay()
    torch.cuda.synchronize()
    got_o, got_s = out.clone(), s1.clone()
    nbytes = lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(a))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    stream = ctypes.c_void_p(torch.cuda.current_stream(gpu).cuda_stream)
    assert lib.ft_attn_colstats_fwd(ctypes.byref(a), s1.data_ptr(), None, ws.data_ptr(), nbytes, stream) == _lib.FT_OK
    torch.cuda.synchronize()
    assert torch.equal(got_o, out) and torch.equal(got_s, s1)


def test_static_scratch_entry_point_limits_and_argument_checks(gpu):
  lib = _lib.load()
  limit = 8 << 20
  st = FtStrides(8 * 2 * 128, 2 * 128, 128)
  # B * H * Sq * 4 bytes of normalisers just beyond the buffer: refused before anything is launched
  B, H, S = 1, 2, limit // (2 * 4) + 1
  big = FtAttnArgs(0x1000, 0x2000, 0x3000, 0x4000, FtStrides(S * 256, 256, 128), FtStrides(S * 256, 256, 128),
                   FtStrides(S * 256, 256, 128), FtStrides(S * 256, 256, 128), B, H, S, S, 128, _lib.FT_F16, _lib.FT_CAUSAL, 0)
  assert lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(big)) > limit
  assert lib.ft_attn_colstats_fwd_static(ctypes.byref(big), 0x5000, None, None) == _lib.FT_EWORKSPACE
  assert b"static buffer holds 8388608" in lib.ft_last_error()
  small = FtAttnArgs(0x1000, 0x2000, 0x3000, 0x4000, st, st, st, st, 1, 2, 8, 8, 128, _lib.FT_F16, _lib.FT_CAUSAL, 0)
  assert lib.ft_attn_colstats_fwd_static(ctypes.byref(small), None, None, None) == _lib.FT_EINVAL      # colsum missing
  small.D = 96
  assert lib.ft_attn_colstats_fwd_static(ctypes.byref(small), 0x5000, None, None) == _lib.FT_EUNSUPPORTED
