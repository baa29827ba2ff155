"""Independent fp64 definitions of the workloads, written from the mathematics (explicit loops over
batch and head, numpy float64, no shared code with `oracle/`), used only to pin the oracle on tiny
shapes: a dropped term, wrong sign, wrong axis or off-by-one mask in the oracle fails against these."""
import numpy as np


def _probs(q, k, b, h):
  Sq, Skv, D = q.shape[1], k.shape[1], q.shape[3]
  s = q[b, :, h, :].astype(np.float64) @ k[b, :, h, :].astype(np.float64).T / np.sqrt(D)
  for i in range(Sq):
    for j in range(Skv):
      if j > i + (Skv - Sq):
        s[i, j] = -np.inf
  e = np.exp(s - s.max(axis=1, keepdims=True))
  return s, e / e.sum(axis=1, keepdims=True)


def attention_stats(q, k, v, exp_rand=None, tau=1.0):
  """Returns O [B,Sq,H,D], colsum [B,H,Skv], colsumsq [B,H,Skv], kf [B,H,Skv] (None without noise)."""
  q, k, v = (t.numpy() if hasattr(t, "numpy") else t for t in (q, k, v))
  B, Sq, H, D = q.shape
  Skv = k.shape[1]
  O = np.zeros((B, Sq, H, D)); cs = np.zeros((B, H, Skv)); cq = np.zeros((B, H, Skv))
  kf = None if exp_rand is None else np.zeros((B, H, Skv))
  for b in range(B):
    for h in range(H):
      s, p = _probs(q, k, b, h)
      O[b, :, h, :] = p @ v[b, :, h, :].astype(np.float64)
      cs[b, h] = p.sum(axis=0)
      cq[b, h] = (p * p).sum(axis=0)
      if exp_rand is not None:
        e = exp_rand[b, h].numpy().astype(np.float64) if hasattr(exp_rand, "numpy") else exp_rand[b, h]
        z = (s - np.log(e)) / tau
        w = np.exp(z - z.max(axis=1, keepdims=True))
        kf[b, h] = (w / w.sum(axis=1, keepdims=True)).sum(axis=0)
  return O, cs, cq, kf


def ea(q, k, v):
  q, k, v = (t.numpy().astype(np.float64) for t in (q, k, v))
  B, S, H, D = q.shape
  O = np.zeros((B, S, H, D))
  for b in range(B):
    for h in range(H):
      Q, K, V = q[b, :, h], k[b, :, h], v[b, :, h]
      qs = np.exp(Q) / np.exp(Q).sum(axis=1, keepdims=True)      # over channels
      ks = np.exp(K) / np.exp(K).sum(axis=0, keepdims=True)      # over tokens
      O[b, :, h] = qs @ (ks.T @ V)
  return O


def sima(q, k, v, normalize_q=True):
  q, k, v = (t.numpy().astype(np.float64) for t in (q, k, v))
  B, S, H, D = q.shape
  O = np.zeros((B, S, H, D))
  for b in range(B):
    for h in range(H):
      Q, K, V = q[b, :, h], k[b, :, h], v[b, :, h]
      kh = K / np.abs(K).sum(axis=0, keepdims=True)
      qh = Q / np.abs(Q).sum(axis=0, keepdims=True) if normalize_q else Q
      O[b, :, h] = qh @ (kh.T @ V)
  return O


def linear_block(core, x, w_qkv, b_qkv, w_out, b_out, H, **kw):
  """y[b,s,m] = sum_c core(q,k,v)[b,s,c] w_out[m,c] + b_out[m] with qkv[b,s,n] = sum_c x[b,s,c] w_qkv[n,c] + b_qkv[n],
  q/k/v = columns [0,C) / [C,2C) / [2C,3C) of qkv, head h = channels [h D, (h+1) D).  fp64, no intermediate
  rounding; index form (einsum subscripts), independent of the oracle's matmul / split / reshape calls."""
  import torch
  x64, wq, bq, wo, bo = (t.numpy().astype(np.float64) for t in (x, w_qkv, b_qkv, w_out, b_out))
  B, S, C = x64.shape
  D = C // H
  qkv = np.einsum("bsc,nc->bsn", x64, wq) + bq[None, None, :]
  parts = []
  for i in range(3):
    t = np.zeros((B, S, H, D))
    for h in range(H):
      t[:, :, h, :] = qkv[:, :, i * C + h * D:i * C + (h + 1) * D]
    parts.append(torch.from_numpy(t))
  o = core(*parts, **kw)            # the fp64 brute-force cores above take any float tensors
  flat = np.zeros((B, S, C))
  for h in range(H):
    flat[:, :, h * D:(h + 1) * D] = o[:, :, h, :]
  return np.einsum("bsc,mc->bsm", flat, wo) + bo[None, None, :]


def avg_pool_same(x, kernel):
  """Stride-1 window mean over the last axis with kernel // 2 zeros on both sides, divisor = kernel."""
  x = np.asarray(x, dtype=np.float64)
  pad = kernel // 2
  out = np.zeros_like(x)
  n = x.shape[-1]
  for j in range(n):
    acc = 0.0
    for t in range(-pad, pad + 1):
      if 0 <= j + t < n:
        acc = acc + x[..., j + t]
    out[..., j] = acc / kernel
  return out


def corm_ratio(q, k, thr):
  """max over query rows of p_ij / thr_ij, [B,H,Skv] float64 (thr: [Sq,Skv])."""
  q, k = (t.numpy() if hasattr(t, "numpy") else t for t in (q, k))
  thr = thr.numpy().astype(np.float64) if hasattr(thr, "numpy") else thr
  B, Sq, H, _ = q.shape
  out = np.zeros((B, H, k.shape[1]))
  for b in range(B):
    for h in range(H):
      _, p = _probs(q, k, b, h)
      out[b, h] = (p / thr).max(axis=0)
  return out


def softcap_attention(q, k, v, cap):
  """O of attention whose scaled logits are replaced by cap * tanh(logit / cap), [B,Sq,H,D] float64."""
  q, k, v = (t.numpy() if hasattr(t, "numpy") else t for t in (q, k, v))
  B, Sq, H, D = q.shape
  Skv = k.shape[1]
  O = np.zeros((B, Sq, H, D))
  for b in range(B):
    for h in range(H):
      s = q[b, :, h, :].astype(np.float64) @ k[b, :, h, :].astype(np.float64).T / np.sqrt(D)
      s = cap * np.tanh(s / cap)
      for i in range(Sq):
        for j in range(Skv):
          if j > i + (Skv - Sq):
            s[i, j] = -np.inf
      e = np.exp(s - s.max(axis=1, keepdims=True))
      O[b, :, h, :] = (e / e.sum(axis=1, keepdims=True)) @ v[b, :, h, :].astype(np.float64)
  return O


def rounding_tie_slack(q, k, weights, tau=1.0, power=1, near=1e-3):
  """How far a per-key score may move because QK^T values sit on fp16 rounding ties: [B,H,Skv], relative.

  The reference rounds QK^T to fp16.  With fp16 inputs the exact dot product is often within 1e-4 ulp of the
  midpoint of two fp16 values, and the order of the fp32 accumulation (torch's CPU matmul, an exact sum rounded
  once, an MFMA) then decides which neighbour it becomes: every one of them is the reference's definition.  The
  neighbour changes the logit by one fp16 ulp u of the raw product, the weight exp(logit / tau) of that pair by
  d = exp(u / (sqrt(D) tau)) - 1, and through the row's normaliser every other weight of the row by w d, w being
  the probability of the pair; a key whose column is dominated by such a row moves with it.
  weights: [B,H,Sq,Skv] fp32, the row-normalised probabilities whose `power`-th powers sum down the columns to
  the score."""
  q, k = (t.numpy().astype(np.float64) for t in (q, k))
  w = weights.numpy().astype(np.float64)
  B, Sq, H, D = q.shape
  out = np.zeros(w.shape[:2] + (w.shape[3],))
  for b in range(B):
    for h in range(H):
      s = q[b, :, h, :] @ k[b, :, h, :].T                      # exact: fp16 products and their sums fit in fp64
      r = s.astype(np.float16).astype(np.float64)              # the nearest fp16 value
      sp = np.spacing(np.abs(r).astype(np.float16)).astype(np.float64)
      dist = np.abs(np.abs(s - r) - sp / 2) / sp               # distance to the midpoint next to it, in ulps
      d = np.where((dist < near) & (w[b, h] > 0), np.expm1(sp / (np.sqrt(D) * tau)), 0.0)
      own = np.expm1(power * np.log1p(d))                      # the pair's own term
      row = power * (w[b, h] * d).sum(axis=1, keepdims=True)   # every term of a row with a tie in it
      wp = w[b, h] ** power
      col = wp.sum(axis=0)
      out[b, h] = (wp * (own + row)).sum(axis=0) / np.where(col > 0, col, 1.0)
  return out
