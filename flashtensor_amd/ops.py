"""Torch-facing operators over the C ABI: one function per fused workload.

Call convention of the reference's emitted kernel wrapper (lib/Translate/to_triton.cpp:540-609): positional
torch tensors in, results allocated with torch.empty on the device of the first argument and returned
(a tuple when there are several), launch on the current stream, no synchronisation.  Torch is used for
device memory and the stream handle only; all arithmetic happens in libflashtensor_hip, reached through the
pybind11 module ft_ffi (csrc/ffi_kernels.cpp, the counterpart of the reference's ffi/ layer): bad arguments
raise ValueError, everything else RuntimeError, as std::invalid_argument / std::runtime_error do there
(ffi/passes.cpp:81-83).
"""
import torch

from . import _lib

_DTYPES = {torch.float16: _lib.FT_F16, torch.bfloat16: _lib.FT_BF16}
_LIN_DTYPES = {**_DTYPES, torch.float32: _lib.FT_F32}  # the linear cores also take the .mlir's own fp32


def _k():
  return _lib.ffi().kernels


def _stream(t):
  return torch.cuda.current_stream(t.device).cuda_stream


def _check_qkv(q, k, v, dtypes=_DTYPES):
  for i, t in enumerate((q, k, v)):
    if not isinstance(t, torch.Tensor):
      raise RuntimeError(f"arg {i} need a torch.Tensor but got {type(t).__name__}")
    if t.dim() != 4:
      raise RuntimeError(f"arg {i} need shape [B, S, H, D] but got {tuple(t.shape)}")
    if not t.is_cuda:
      raise RuntimeError(f"arg {i} need a GPU tensor but got device {t.device}")
    if t.dtype != q.dtype or t.device != q.device:
      raise RuntimeError(f"arg {i} need dtype {q.dtype} on {q.device} but got {t.dtype} on {t.device}")
  if q.dtype not in dtypes:
    raise RuntimeError(f"arg 0 need dtype {' or '.join(str(d).split('.')[-1] for d in dtypes)} but got {q.dtype}")
  B, Sq, H, D = q.shape
  Hkv = k.shape[2]
  if tuple(k.shape) != (B, k.shape[1], Hkv, D) or Hkv < 1 or H % Hkv != 0:
    raise RuntimeError(f"arg 1 need shape {(B, k.shape[1], 'a divisor of ' + str(H), D)} but got {tuple(k.shape)}")
  if tuple(v.shape) != tuple(k.shape):
    raise RuntimeError(f"arg 2 need shape {tuple(k.shape)} but got {tuple(v.shape)}")


def _dense_last(t):
  """The kernels read rows of contiguous elements; a tensor whose last axis is strided is refused (as the C
  ABI refuses it) rather than copied behind the caller's back."""
  if t.stride(-1) != 1 and t.shape[-1] != 1:
    raise ValueError(f"need a contiguous last axis but got strides {tuple(t.stride())} for shape {tuple(t.shape)}")
  return t


def _args(q, k, v, o, flags):
  B, Sq, H, D = q.shape
  return _k().AttnArgs(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), q.stride()[:3], k.stride()[:3], v.stride()[:3],
                       o.stride()[:3], B, H, Sq, k.shape[1], D, _LIN_DTYPES[q.dtype], flags, k.shape[2])


def _flags(causal, fast_logits):
  return (_lib.FT_CAUSAL if causal else 0) | (_lib.FT_FAST_LOGITS if fast_logits else 0)


def _prep(q, k, v, dtypes=_DTYPES):
  _check_qkv(q, k, v, dtypes)
  return _dense_last(q), _dense_last(k), _dense_last(v)


def attn(q, k, v, causal=True, fast_logits=False, return_lse=False):
  """Attn.forward (cases/kernels/attn.py:18-34): q [B,S,H,D], k,v [B,Skv,Hkv,D] -> out [B,Sq,H,D].  With
  Hkv < H query head h attends to k/v head h // (H // Hkv), the grouping of cases/attn.py:29-31."""
  q, k, v = _prep(q, k, v)
  out = torch.empty_like(q, memory_format=torch.contiguous_format)
  lse = torch.empty(q.shape[0], q.shape[2], q.shape[1], dtype=torch.float32, device=q.device) if return_lse else None
  _k().attn_fwd(_args(q, k, v, out, _flags(causal, fast_logits)), lse.data_ptr() if return_lse else 0, _stream(q))
  return (out, lse) if return_lse else out


def _colstats(q, k, v, want_sq, causal, fast_logits):
  q, k, v = _prep(q, k, v)
  ffi = _k()
  B, Sq, H, D = q.shape
  Skv = k.shape[1]
  out = torch.empty_like(q, memory_format=torch.contiguous_format)
  s1 = torch.empty(B, k.shape[2], Skv, dtype=torch.float32, device=q.device)  # per k/v head (group mean when grouped)
  s2 = torch.empty(B, H, Skv, dtype=torch.float32, device=q.device) if want_sq else None
  a = _args(q, k, v, out, _flags(causal, fast_logits))
  nbytes = ffi.workspace_bytes(_lib.FT_OP_COLSTATS, a)
  ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
  ffi.attn_colstats_fwd(a, s1.data_ptr(), s2.data_ptr() if want_sq else 0, ws.data_ptr(), nbytes, _stream(q))
  return (out, s1, s2) if want_sq else (out, s1)


def h2o(q, k, v, causal=True, fast_logits=False):
  """H2O.forward (cases/kernels/h2o.py:18-38) -> (out, h2o_score [B,Hkv,Skv] fp32); under grouped queries
  the probabilities are averaged over each group's query heads before the sum (cases/attn_h2o.py:42-47)."""
  return _colstats(q, k, v, False, causal, fast_logits)


def roco(q, k, v, causal=True, fast_logits=False):
  """RoCo.forward (cases/kernels/roco.py:18-48) -> (out, roco_score, roco_sq_score), scores [B,H,Skv] fp32."""
  return _colstats(q, k, v, True, causal, fast_logits)


def keyformer(q, k, v, exp_rand=None, tau=1.5, seed=0, causal=True, fast_logits=False):
  """KeyFormer.forward (cases/kernels/kf.py:19-42) -> (out, kf_score [B,H,Skv] fp32).
  exp_rand [B,H,Sq,Skv] fp32 is the reference's noise input; None draws it in-kernel from `seed`."""
  q, k, v = _prep(q, k, v)
  ffi = _k()
  B, Sq, H, D = q.shape
  Skv = k.shape[1]
  noise = ffi.Noise(0, 0, 0, 0, int(seed) & 0xFFFFFFFFFFFFFFFF)
  if exp_rand is not None:
    if tuple(exp_rand.shape) != (B, H, Sq, Skv):
      raise RuntimeError(f"arg 3 need shape {(B, H, Sq, Skv)} but got {tuple(exp_rand.shape)}")
    if exp_rand.dtype != torch.float32 or exp_rand.device != q.device:
      raise RuntimeError(f"arg 3 need dtype torch.float32 on {q.device} but got {exp_rand.dtype} on {exp_rand.device}")
    exp_rand = _dense_last(exp_rand)
    noise = ffi.Noise(exp_rand.data_ptr(), exp_rand.stride(0), exp_rand.stride(1), exp_rand.stride(2), 0)
  out = torch.empty_like(q, memory_format=torch.contiguous_format)
  score = torch.empty(B, H, Skv, dtype=torch.float32, device=q.device)
  a = _args(q, k, v, out, _flags(causal, fast_logits))
  nbytes = ffi.workspace_bytes(_lib.FT_OP_KEYFORMER, a)
  ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
  ffi.keyformer_fwd(a, noise, float(tau), score.data_ptr(), ws.data_ptr(), nbytes, _stream(q))
  return out, score


def snapkv(q, k, v, kernel_size=5, causal=True, fast_logits=False):
  """SnapKV.forward (cases/kernels/snapkv.py:19-43) -> (out, snapkv_score [B,H,Skv] fp32): the H2O column
  sums smoothed by a stride-1 average pool of odd width `kernel_size` over the key axis."""
  out, score = _colstats(q, k, v, False, causal, fast_logits)
  B, H, Skv = score.shape
  pooled = torch.empty_like(score)
  _k().avgpool1d(score.data_ptr(), B * H, Skv, int(kernel_size), pooled.data_ptr(), _stream(q))
  return out, pooled


def corm(q, k, v, corm_mask=None, causal=True, fast_logits=False, return_margin=False):
  """Corm.forward (cases/kernels/corm.py:18-40) -> (out, corm_score [B,H,Skv] bool): key j is kept when some
  query row gives it a probability >= corm_mask[i, j].  corm_mask [Sq,Skv] fp32 is the reference's input;
  None applies its prepare() recipe 1 / (i + 1) (corm.py:47-49) without reading a tensor."""
  q, k, v = _prep(q, k, v)
  ffi = _k()
  B, Sq, H, D = q.shape
  Skv = k.shape[1]
  mask_ptr, mask_stride = 0, 0
  if corm_mask is not None:
    if tuple(corm_mask.shape) != (Sq, Skv):
      raise RuntimeError(f"arg 3 need shape {(Sq, Skv)} but got {tuple(corm_mask.shape)}")
    if corm_mask.dtype != torch.float32 or corm_mask.device != q.device:
      raise RuntimeError(f"arg 3 need dtype torch.float32 on {q.device} but got {corm_mask.dtype} on {corm_mask.device}")
    corm_mask = _dense_last(corm_mask)
    mask_ptr, mask_stride = corm_mask.data_ptr(), corm_mask.stride(0)
  out = torch.empty_like(q, memory_format=torch.contiguous_format)
  keep = torch.empty(B, H, Skv, dtype=torch.uint8, device=q.device)
  margin = torch.empty(B, H, Skv, dtype=torch.float32, device=q.device) if return_margin else None
  a = _args(q, k, v, out, _flags(causal, fast_logits))
  nbytes = ffi.workspace_bytes(_lib.FT_OP_CORM, a)
  ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
  ffi.corm_fwd(a, mask_ptr, mask_stride, keep.data_ptr(), margin.data_ptr() if return_margin else 0, ws.data_ptr(), nbytes,
               _stream(q))
  keep = keep.view(torch.bool)
  return (out, keep, margin) if return_margin else (out, keep)


def gemma2(q, k, v, softcap=50.0, causal=True, fast_logits=False):
  """Gemma2.forward (cases/kernels/gemma2.py:19-39): attention with logits softcap * tanh(logit / softcap)."""
  q, k, v = _prep(q, k, v)
  out = torch.empty_like(q, memory_format=torch.contiguous_format)
  _k().attn_softcap_fwd(_args(q, k, v, out, _flags(causal, fast_logits)), float(softcap), 0, _stream(q))
  return out


def _linattn(q, k, v, kind, normalize_q, out_dtype):
  q, k, v = _prep(q, k, v, _LIN_DTYPES)
  if q.shape[3] == 32:  # head_dim 32 runs as pairs of adjacent heads: heads must lie 32 elements apart
    for i, t in enumerate((q, k, v)):
      if t.stride(2) != 32:
        raise ValueError(f"arg {i} with head_dim 32 need heads stored 32 elements apart but got head stride {t.stride(2)}")
  ffi = _k()
  out_dtype = out_dtype or q.dtype
  if out_dtype not in (q.dtype, torch.float32):
    raise RuntimeError(f"out_dtype need {q.dtype} or float32 but got {out_dtype}")
  out = torch.empty(q.shape, dtype=out_dtype, device=q.device)
  a = _args(q, k, v, out, 0)
  nbytes = ffi.workspace_bytes(kind, a)
  ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
  ffi.linattn_fwd(a, kind, int(bool(normalize_q)), _LIN_DTYPES[out_dtype], ws.data_ptr(), nbytes, _stream(q))
  return out


def ea(q, k, v, out_dtype=None):
  """EA core (bench/ea.mlir:13-17): softmax(Q, dim=D) (softmax(K, dim=S)^T V); q,k,v [B,S,H,D] -> [B,S,H,D]."""
  return _linattn(q, k, v, _lib.FT_OP_EA, True, out_dtype)


def sima(q, k, v, normalize_q=True, out_dtype=None):
  """SimA core (bench/sima.mlir:13-17): L1-normalised Q, K over S per channel, O = Qh (Kh^T V).
  normalize_q=False multiplies by the raw Q as line 17 of the .mlir does."""
  return _linattn(q, k, v, _lib.FT_OP_SIMA, normalize_q, out_dtype)


def _linattn_block(x, w_qkv, b_qkv, w_out, b_out, head_num, kind, normalize_q):
  tensors = [("x", x), ("w_qkv", w_qkv), ("b_qkv", b_qkv), ("w_out", w_out), ("b_out", b_out)]
  for i, (name, t) in enumerate(tensors):
    if t is None and name.startswith("b_"):
      continue
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
      raise RuntimeError(f"arg {i} ({name}) need a GPU tensor")
    if t.dtype != x.dtype:
      raise RuntimeError(f"arg {i} ({name}) need {x.dtype} but got {t.dtype}")
  if x.dim() != 3 or x.shape[2] % head_num:
    raise ValueError(f"x need [B,S,C] with C a multiple of head_num={head_num} but got {tuple(x.shape)}")
  B, S, C = x.shape
  if tuple(w_qkv.shape) != (3 * C, C) or tuple(w_out.shape) != (C, C):
    raise ValueError(f"weights need [{3 * C},{C}] and [{C},{C}] but got {tuple(w_qkv.shape)} and {tuple(w_out.shape)}")
  if (b_qkv is not None and tuple(b_qkv.shape) != (3 * C,)) or (b_out is not None and tuple(b_out.shape) != (C,)):
    raise ValueError(f"biases need [{3 * C}] and [{C}]")
  ffi = _k()
  for i, (name, t) in enumerate(tensors):
    if t is not None and not t.is_contiguous():
      raise ValueError(f"arg {i} ({name}) need a contiguous tensor but got strides {tuple(t.stride())}")
  y = torch.empty_like(x)
  if x.dtype not in _LIN_DTYPES:
    raise RuntimeError(f"arg 0 (x) need float16, bfloat16 or float32 but got {x.dtype}")
  dt = _LIN_DTYPES[x.dtype]
  a = ffi.LinBlockArgs(x.data_ptr(), w_qkv.data_ptr(), 0 if b_qkv is None else b_qkv.data_ptr(), w_out.data_ptr(),
                       0 if b_out is None else b_out.data_ptr(), y.data_ptr(), B, S, head_num, C // head_num, dt)
  nbytes = ffi.linattn_block_workspace_bytes(a, kind)
  if nbytes == 0:
    raise RuntimeError(f"libflashtensor_hip: {ffi.last_error()}")
  ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
  ffi.linattn_block_fwd(a, kind, int(bool(normalize_q)), ws.data_ptr(), nbytes, _stream(x))
  return y


def ea_block(x, w_qkv, b_qkv, w_out, b_out, head_num):
  """The whole function of bench/ea.mlir:2-23: q/k/v Linear, split into heads, EA core, output Linear.
  x [B,S,C], w_qkv [3C,C], b_qkv [3C], w_out [C,C], b_out [C] -> [B,S,C]."""
  return _linattn_block(x, w_qkv, b_qkv, w_out, b_out, head_num, _lib.FT_OP_EA, True)


def sima_block(x, w_qkv, b_qkv, w_out, b_out, head_num, normalize_q=True):
  """The whole function of bench/sima.mlir:2-23 (normalize_q as for `sima`)."""
  return _linattn_block(x, w_qkv, b_qkv, w_out, b_out, head_num, _lib.FT_OP_SIMA, normalize_q)


def topk(score, k):
  """Indices [..., k] (int64) of the k largest entries along the last axis, descending."""
  if score.dtype != torch.float32 or not score.is_cuda:
    raise RuntimeError(f"arg 0 need a float32 GPU tensor but got {score.dtype} on {score.device}")
  if not score.is_contiguous():
    raise ValueError(f"arg 0 need a contiguous tensor but got strides {tuple(score.stride())}")
  s = score
  S = s.shape[-1]
  rows = s.numel() // S
  idx = torch.empty(*s.shape[:-1], k, dtype=torch.int64, device=s.device)
  _k().topk(s.data_ptr(), rows, S, int(k), idx.data_ptr(), _stream(s))
  return idx


def seeded_exp_rand(B, H, Sq, Skv, seed, device):
  """The noise tensor the seeded KeyFormer mode draws, materialised on `device` ("cpu" uses the host twin)."""
  device = torch.device(device)
  out = torch.empty(B, H, Sq, Skv, dtype=torch.float32, device=device)
  seed = int(seed) & 0xFFFFFFFFFFFFFFFF
  if device.type == "cpu":
    _k().noise_exp_fill_host(out.data_ptr(), B, H, Sq, Skv, seed)
  else:
    _k().noise_exp_fill(out.data_ptr(), B, H, Sq, Skv, seed, _stream(out))
  return out
