"""CPU restatement of the reference's eager workloads (the numerical definition of the hot path).

TEST INFRASTRUCTURE (see `oracle/__init__.py`): the checker for the HIP kernels and the CPU baseline
that `bench.py` times.  Never imported by the product package.

Same torch ops, same order, same dtype at every step as the reference, so the rounding points are
the reference's: QK^T rounded to fp16, divided by sqrt(D) in fp16, fp16 mask added, softmax in fp32,
P rounded to fp16 before PV.

How each function is pinned (tests/test_oracle_pins.py, tests/test_oracle_golden.py):
  attn_forward       torch's F.scaled_dot_product_attention(is_causal=True) in fp32; row 0 == v[0]
                     bit-exact; q == 0 -> prefix means of V; fp64 brute force for S <= 64.
  h2o_forward        sum_j score_j == Sq; q == 0 -> score_j = H_S - H_j (harmonic numbers);
                     score_{S-1} == p_{S-1,S-1}; fp64 brute force.
  roco_forward       sums as h2o; q == 0 -> sumsq_j = sum_{i>=j} (i+1)^-2; 0 <= sumsq <= sum.
  keyformer_forward  exp_rand == 1, tau == 1 -> kf_score == h2o score; tau -> inf -> uniform closed
                     form; sum_j == Sq; fp64 brute force with random noise.
  ea_forward         V == c -> O == c; Q == K == 0 -> O = mean_s V; fp64 brute force.
  sima_forward       sum_s |Qhat| == 1; scale invariance in Q and K; fp64 brute force.
  snapkv_forward     kernel_size == 1 -> the H2O score; explicit zero-padded window loop in numpy on
                     top of the fp64 brute-force column sums; interior windows of a constant score.
  corm_forward       key 0 is always kept (p_00 == 1 >= 1); q == 0 -> p_ij == 1/(i+1) exactly -> every key
                     kept; an all-ones mask keeps exactly the keys some row attends to with p == 1; fp64
                     brute force away from the decision boundary (corm_margin).
  gemma2_forward     softcap = 512 (a power of two, tanh(y) == y in fp16 for the tiny y) -> attn_forward
                     up to last-bit flips; tiny softcap -> logits ~ 0 -> prefix means of V; fp64 brute
                     force at caps 50 and 2.
  attn2d_forward,    Hkv == H -> attn_forward / h2o_forward on the [1,S,H,D] views, bit-exact; Hkv < H ->
  attn_h2o2d_forward the same functions on k/v heads repeated with repeat_interleave, scores averaged per group;
                     fp64 brute force with explicit h // group indexing; unmasked rows sum to Sq.
  ea_block_forward,  stacked identity weights, zero biases -> the core on (x, x, x), bit-exact; x == 0 -> q, k, v
  sima_block_forward are the bias rows, V constant over tokens -> y == w_out b_v + b_out (EA); fp64 brute force with
                     explicit loops over a non-symmetric weight (a transposed operand or a wrong split order fails).
The reference holds no golden vectors or tests for this path, so none can be checked against; no
function of this file is "parity unpinned".
"""
import math

import torch
import torch.nn.functional as F


def _masked_scores_probs(q, k):
  """Shared prefix of every softmax case (cases/kernels/h2o.py:19-31, identical in attn.py:19-31,
  kf.py:20-32, roco.py:19-37).  q,k: [B,S,H,D].  Returns (scores fp16 masked [B,H,Sq,Skv], probs fp32)."""
  q_len, kv_len = q.shape[1], k.shape[1]
  head_dim = q.shape[3]
  mask = torch.full((1, 1, q_len, kv_len), -torch.inf, device=q.device, dtype=q.dtype)
  mask = torch.triu(mask, diagonal=kv_len - q_len + 1)
  qt = q.transpose(1, 2)
  kt = k.transpose(1, 2)
  scores = torch.matmul(qt, kt.transpose(-2, -1)) / math.sqrt(head_dim)
  scores += mask
  probs = F.softmax(scores.float(), dim=-1)
  return scores, probs


def _out(probs, q, v):
  """cases/kernels/h2o.py:32,38: P rounded to the input dtype, PV, back to [B,Sq,H,D]."""
  B, q_len, H, D = q.shape
  out = torch.matmul(probs.to(q.dtype), v.transpose(1, 2)).transpose(1, 2).contiguous()
  return out.view(B, q_len, H, D)


def attn_forward(q, k, v):
  """Causal softmax attention, cases/kernels/attn.py:18-34.  q,k,v [B,S,H,D] -> out [B,Sq,H,D]."""
  _, probs = _masked_scores_probs(q, k)
  return _out(probs, q, v)


def h2o_forward(q, k, v):
  """H2O, cases/kernels/h2o.py:18-38: attention + per-key accumulated probability
  h2o_score[b,h,j] = sum_i probs[b,h,i,j] (fp32, [B,H,Skv])."""
  _, probs = _masked_scores_probs(q, k)
  out = _out(probs, q, v)
  h2o_score = probs.sum(dim=2)
  return out, h2o_score.view(q.shape[0], q.shape[2], k.shape[1])


def roco_forward(q, k, v):
  """RoCo, cases/kernels/roco.py:18-48 (group_size == 1 branch, asserted at :16): attention + per-key
  sum and sum of squares of the probabilities over query rows (both fp32 [B,H,Skv])."""
  _, probs = _masked_scores_probs(q, k)
  out = _out(probs, q, v)
  roco_score = probs.sum(dim=2)
  roco_sq_score = (probs ** 2).sum(dim=2)
  shp = (q.shape[0], q.shape[2], k.shape[1])
  return out, roco_score.view(shp), roco_sq_score.view(shp)


def keyformer_forward(q, k, v, exp_rand, tau=1.5):
  """KeyFormer, cases/kernels/kf.py:19-42 (tau default :8): attention (unperturbed O) + per-key column
  sum of softmax((masked fp16 scores as fp32 + gumbels) / tau) with gumbels = -log(exp_rand)."""
  scores, probs = _masked_scores_probs(q, k)
  out = _out(probs, q, v)
  gumbels = -exp_rand.log()
  kf_score = (scores.float() + gumbels) / tau
  kf_score = F.softmax(kf_score.float(), dim=-1)
  kf_score = kf_score.sum(dim=2)
  return out, kf_score.view(q.shape[0], q.shape[2], k.shape[1])


def snapkv_forward(q, k, v, kernel_size=5):
  """SnapKV, cases/kernels/snapkv.py:19-43 (kernel_size default :8): attention + the per-key column sum
  of the probabilities smoothed by a stride-1 average pool over keys (zero padding of kernel_size // 2,
  padded positions counted in the divisor: F.avg_pool1d defaults)."""
  _, probs = _masked_scores_probs(q, k)
  out = _out(probs, q, v)
  snapkv_score = probs.sum(dim=2)
  snapkv_score = F.avg_pool1d(snapkv_score, kernel_size=kernel_size, padding=kernel_size // 2, stride=1)
  return out, snapkv_score.view(q.shape[0], q.shape[2], k.shape[1])


def corm_mask_rule(q_len, kv_len):
  """Threshold recipe of Corm.prepare (cases/kernels/corm.py:47-49): row i holds 1 / (i + 1), fp32."""
  rows = torch.arange(1, q_len + 1, dtype=torch.float32).unsqueeze(1)
  return torch.ones(q_len, kv_len, dtype=torch.float32) / rows


def corm_forward(q, k, v, corm_mask):
  """CoRM, cases/kernels/corm.py:18-40: attention + corm_score[b,h,j] = any_i(probs[b,h,i,j] >=
  corm_mask[i,j]) (bool [B,H,Skv]); corm_mask is fp32 [Sq,Skv]."""
  _, probs = _masked_scores_probs(q, k)
  out = _out(probs, q, v)
  corm_score = probs >= corm_mask
  corm_score = corm_score.any(dim=2)
  return out, corm_score.view(q.shape[0], q.shape[2], k.shape[1])


def corm_margin(q, k, corm_mask):
  """max_i probs[b,h,i,j] / corm_mask[i,j] ([B,H,Skv] fp32): corm_score is True iff this is >= 1; its
  distance from 1 tells how far a key is from the decision boundary (used for the comparison rule of
  the parity tests, not part of the reference)."""
  _, probs = _masked_scores_probs(q, k)
  return (probs / corm_mask).amax(dim=2)


def gemma2_forward(q, k, v, softcap=50.0):
  """Gemma2 soft-capped attention, cases/kernels/gemma2.py:19-39 (logit_softcapping default :8): the
  fp16 scores are divided by the cap, passed through tanh and multiplied by the cap again, each step an
  fp16 tensor op, before the mask and the fp32 softmax."""
  q_len, kv_len = q.shape[1], k.shape[1]
  mask = torch.full((1, 1, q_len, kv_len), -torch.inf, device=q.device, dtype=q.dtype)
  mask = torch.triu(mask, diagonal=kv_len - q_len + 1)
  qt = q.transpose(1, 2)
  kt = k.transpose(1, 2)
  scores = torch.matmul(qt, kt.transpose(-2, -1)) / math.sqrt(q.shape[3])
  scores /= softcap
  scores = torch.tanh(scores)
  scores *= softcap
  scores += mask
  probs = F.softmax(scores.float(), dim=-1)
  return _out(probs, q, v)


def _probs_2d(q, k, v, kv_head_num, head_num, head_dim, masked):
  """Shared body of cases/attn.py:20-42,44-63 and cases/attn_h2o.py:19-40,50-66: 2-D activations, grouped
  queries by expanding k/v heads, optional causal mask.  Returns (probs fp32 [H,Sq,Skv], q, v as [H,S,D])."""
  q_len, kv_len = q.shape[0], k.shape[0]
  group_size = head_num // kv_head_num
  q = q.view(q_len, head_num, head_dim)
  k = k.view(kv_len, kv_head_num, head_dim)
  v = v.view(kv_len, kv_head_num, head_dim)
  if group_size > 1:
    k = k[:, :, None, :].expand(kv_len, kv_head_num, group_size, head_dim).reshape(kv_len, head_num, head_dim)
    v = v[:, :, None, :].expand(kv_len, kv_head_num, group_size, head_dim).reshape(kv_len, head_num, head_dim)
  q, k, v = q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)
  scores = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(head_dim)
  if masked:
    mask = torch.full((1, q_len, kv_len), -torch.inf, device=q.device, dtype=scores.dtype)
    scores += torch.triu(mask, diagonal=kv_len - q_len + 1)
  return F.softmax(scores.float(), dim=-1), q, v


def attn2d_forward(q, k, v, kv_head_num, head_num, head_dim, masked=True):
  """cases/attn.py:20-69: q [q_len, H*D], k, v [kv_len, Hkv*D] -> out [q_len, H*D]."""
  probs, qh, vh = _probs_2d(q, k, v, kv_head_num, head_num, head_dim, masked)
  out = torch.matmul(probs.to(qh.dtype), vh).transpose(0, 1).contiguous()
  return out.view(q.shape[0], head_num * head_dim)


def attn_h2o2d_forward(q, k, v, kv_head_num, head_num, head_dim, masked=True):
  """cases/attn_h2o.py:19-81: as attn2d_forward plus h2o_score [Hkv, kv_len] = sum over query rows of the
  probabilities averaged over the query heads of each group (:42-47)."""
  q_len, kv_len = q.shape[0], k.shape[0]
  group_size = head_num // kv_head_num
  probs, qh, vh = _probs_2d(q, k, v, kv_head_num, head_num, head_dim, masked)
  out = torch.matmul(probs.to(qh.dtype), vh).transpose(0, 1).contiguous()
  if group_size > 1:
    h2o_score = probs.reshape(kv_head_num, group_size, q_len, kv_len).mean(dim=1)
  else:
    h2o_score = probs
  h2o_score = h2o_score.sum(dim=1)
  return out.view(q_len, head_num * head_dim), h2o_score.view(kv_head_num, kv_len)


def ea_forward(q, k, v):
  """EA linear-attention core, bench/ea.mlir:13-17 with softmax = exp/sum over `dim`
  (lib/Dialect/Asuka/Transforms/LowerComplexReduce.cpp:21-41): Qs = softmax(Q, dim=D),
  Ks = softmax(K, dim=S), KV = Ks^T V, O = Qs KV.  q,k,v [B,S,H,D] fp16; the reference graph is f32, so
  the internal math is fp32 and O is rounded once to the input dtype."""
  qf, kf, vf = (t.transpose(1, 2).float() for t in (q, k, v))  # [B,H,S,D]
  qs = F.softmax(qf, dim=3)
  ks = F.softmax(kf, dim=2)
  kv = torch.matmul(ks.transpose(-2, -1), vf)  # [B,H,D,D]
  out = torch.matmul(qs, kv)
  return out.transpose(1, 2).contiguous().to(q.dtype)


def sima_forward(q, k, v, normalize_q=True, out_dtype=None):
  """SimA linear-attention core, bench/sima.mlir:13-17 with normalize(Lp=1) = x / sum(|x|) over `dim`,
  keep-dim, signed numerator (LowerComplexReduce.cpp:43-69): Qh = Q/sum_s|Q|, Kh = K/sum_s|K| per
  (b,h,channel), O = Qh (Kh^T V).  normalize_q=False reproduces the .mlir's use of the raw Q at :17."""
  qf, kf, vf = (t.transpose(1, 2).float() for t in (q, k, v))
  kh = kf / kf.abs().sum(dim=2, keepdim=True)
  qh = qf / qf.abs().sum(dim=2, keepdim=True) if normalize_q else qf
  kv = torch.matmul(kh.transpose(-2, -1), vf)
  out = torch.matmul(qh, kv)
  return out.transpose(1, 2).contiguous().to(out_dtype or q.dtype)


def _linear16(x, w, b):
  """A Linear as the .mlir writes it (transpose, dot, add: bench/ea.mlir:3-5 and :20-22), evaluated in fp32
  from 16-bit operands and rounded once to the operand dtype: the rounding points of a 16-bit GEMM with
  fp32 accumulation and a fused bias."""
  y = torch.matmul(x.float(), w.float().transpose(0, 1))
  if b is not None:
    y = y + b.float()
  return y.to(x.dtype)


def _block(core, x, w_qkv, b_qkv, w_out, b_out, head_num, **kw):
  B, S, C = x.shape
  qkv = _linear16(x, w_qkv, b_qkv)                                          # ea.mlir:3-5
  q, k, v = (t.reshape(B, S, head_num, C // head_num) for t in qkv.split(C, dim=2))  # :6-9 (core transposes, :10-12)
  o = core(q, k, v, **kw)                                                   # :13-19
  return _linear16(o.reshape(B, S, C), w_out, b_out)                        # :20-22


def ea_block_forward(x, w_qkv, b_qkv, w_out, b_out, head_num):
  """The whole function of bench/ea.mlir:2-23 on 16-bit tensors (the graph itself is f32; q/k/v, the core's
  result and y are the 16-bit tensors between the stages)."""
  return _block(ea_forward, x, w_qkv, b_qkv, w_out, b_out, head_num)


def sima_block_forward(x, w_qkv, b_qkv, w_out, b_out, head_num, normalize_q=True):
  """The whole function of bench/sima.mlir:2-23."""
  return _block(sima_forward, x, w_qkv, b_qkv, w_out, b_out, head_num, normalize_q=normalize_q)


def prepare_block_inputs(B, S, H, D, seed=0, dtype=torch.float16):
  """x ~ N(0,1); weights ~ N(0,1/C) so that q, k, v come out ~ N(0,1) as in the core's own recipe; biases 0.1 N(0,1)."""
  g = torch.Generator(device="cpu")
  g.manual_seed(seed)
  C = H * D
  x = torch.randn(B, S, C, dtype=dtype, generator=g)
  w_qkv = (torch.randn(3 * C, C, generator=g) / C ** 0.5).to(dtype)
  b_qkv = (0.1 * torch.randn(3 * C, generator=g)).to(dtype)
  w_out = (torch.randn(C, C, generator=g) / C ** 0.5).to(dtype)
  b_out = (0.1 * torch.randn(C, generator=g)).to(dtype)
  return x, w_qkv, b_qkv, w_out, b_out


# ---------------------------------------------------------------------------------------------------
# Input recipes and epilogues


def prepare_inputs(B, S, H, D, seed=0, dtype=torch.float16, kv_len=None):
  """Input recipe of every case's prepare() (cases/kernels/attn.py:36-39): q, k, v ~ N(0,1) drawn in
  that order in the target dtype, here from the seeded CPU generator (cases/attn.py:89)."""
  g = torch.Generator(device="cpu")
  g.manual_seed(seed)
  kv_len = S if kv_len is None else kv_len
  q = torch.randn(B, S, H, D, dtype=dtype, generator=g)
  k = torch.randn(B, kv_len, H, D, dtype=dtype, generator=g)
  v = torch.randn(B, kv_len, H, D, dtype=dtype, generator=g)
  return q, k, v


def prepare_exp_rand(B, H, Sq, Skv, seed=0):
  """Noise recipe of KeyFormer.prepare (cases/kernels/kf.py:48): 1 + |N(0,1)|, fp32."""
  g = torch.Generator(device="cpu")
  g.manual_seed(seed + 7919)
  return 1 + torch.randn(B, H, Sq, Skv, dtype=torch.float32, generator=g).abs()


def heavy_hitters(score, k):
  """Top-k key indices per head of a [B,H,S] score, descending by score.  Not in the reference (its
  H2O case stops at the score, cases/kernels/h2o.py:34-38); the measured configuration asks for k=S/8."""
  return torch.topk(score, k, dim=-1, largest=True, sorted=True).indices


def roco_mean_var(roco_score, roco_sq_score, q_len):
  """Mean and (population) variance over the q_len query rows from RoCo's sum and sum of squares."""
  mean = roco_score / q_len
  return mean, roco_sq_score / q_len - mean * mean


def chunked_over_heads(fn, tensors, head_chunk, extra=(), **kw):
  """Evaluate fn on slices of the head axis (dim 2 of q/k/v; dim 1 of [B,H,...] extras and results) and
  concatenate: heads are independent, so results are identical while peak memory is bounded."""
  H = tensors[0].shape[2]
  pieces = []
  for h0 in range(0, H, head_chunk):
    sl = slice(h0, min(H, h0 + head_chunk))
    args = [t[:, :, sl].contiguous() for t in tensors] + [e[:, sl] for e in extra]
    res = fn(*args, **kw)
    pieces.append(res if isinstance(res, tuple) else (res,))
  outs = []
  for idx in range(len(pieces[0])):
    parts = [p[idx] for p in pieces]
    # O is [B,S,H,D] (head axis 2); scores are [B,H,S] (head axis 1)
    outs.append(torch.cat(parts, dim=2 if parts[0].dim() == 4 else 1))
  return outs[0] if len(outs) == 1 else tuple(outs)
