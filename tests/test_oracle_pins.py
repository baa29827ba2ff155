"""Pins the CPU oracle: library routine, closed forms, invariants and fp64 brute force (CPU only).

The reference has no tests, fixtures or golden vectors for this path, so the oracle is pinned by what
the mathematics fixes.  Each check is chosen so that a plausible mistake (mask off by one, wrong softmax
axis, sum over the wrong dimension, dropped 1/tau, sign of the Gumbel term, transposed K^T V) fails it.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from tests import brute


def _inputs(B=1, S=64, H=2, D=64, seed=0, kv_len=None):
  return oracle.prepare_inputs(B, S, H, D, seed=seed, kv_len=kv_len)


# ------------------------------------------------------------------ attention output

@pytest.mark.parametrize("S,D", [(64, 64), (128, 128), (96, 128)])
def test_attn_matches_sdpa_fp32(S, D):
  q, k, v = _inputs(S=S, D=D)
  out = oracle.attn_forward(q, k, v)
  ref = F.scaled_dot_product_attention(q.transpose(1, 2).float(), k.transpose(1, 2).float(),
                                       v.transpose(1, 2).float(), is_causal=True).transpose(1, 2)
  assert out.dtype == torch.float16 and out.shape == q.shape
  assert (out.float() - ref).abs().max() < 4e-3  # fp16 rounding points of the eager definition


def test_attn_row0_is_v0_bit_exact():
  q, k, v = _inputs(S=128, D=128)
  out = oracle.attn_forward(q, k, v)
  assert torch.equal(out[:, 0], v[:, 0])


def test_attn_zero_q_gives_prefix_means():
  q, k, v = _inputs(S=64, D=64)
  out = oracle.attn_forward(torch.zeros_like(q), k, v)
  ref = v.float().cumsum(dim=1) / torch.arange(1, 65).view(1, -1, 1, 1)
  assert (out.float() - ref).abs().max() < 2e-3


def test_attn_rectangular_mask_offset():
  # Sq < Skv: row i sees keys j <= i + (Skv - Sq) (triu diagonal = Skv - Sq + 1)
  q, k, v = _inputs(S=32, D=64, kv_len=80)
  out = oracle.attn_forward(q, k, v)
  O, _, _, _ = brute.attention_stats(q, k, v)
  assert np.abs(out.float().numpy() - O).max() < 4e-3


# ------------------------------------------------------------------ column statistics

def test_h2o_brute_force_and_invariants():
  q, k, v = _inputs(B=2, S=64, H=2, D=64, seed=3)
  out, score = oracle.h2o_forward(q, k, v)
  O, cs, _, _ = brute.attention_stats(q, k, v)
  assert score.dtype == torch.float32 and score.shape == (2, 2, 64)
  assert np.abs(out.float().numpy() - O).max() < 4e-3
  assert np.abs(score.numpy() - cs).max() / np.abs(cs).max() < 2e-3
  # rows of P sum to one => total mass is Sq per (b,h)
  assert torch.allclose(score.sum(-1), torch.full((2, 2), 64.0), rtol=1e-5)
  # the last key is seen by the last query only: score_{S-1} = p_{S-1,S-1}
  scores, probs = oracle.cases._masked_scores_probs(q, k)
  assert torch.equal(score[..., -1], probs[..., -1, -1])


def test_h2o_zero_q_harmonic_closed_form():
  S = 96
  q, k, v = _inputs(S=S, D=64)
  _, score = oracle.h2o_forward(torch.zeros_like(q), k, v)
  # uniform causal probs: p_ij = 1/(i+1) for j <= i  =>  score_j = sum_{i>=j} 1/(i+1) = H_S - H_j
  harm = np.concatenate([[0.0], np.cumsum(1.0 / np.arange(1, S + 1))])
  ref = harm[S] - harm[:S]
  assert np.abs(score[0, 0].numpy() - ref).max() < 1e-5


def test_roco_closed_form_and_bounds():
  S = 80
  q, k, v = _inputs(S=S, D=64, seed=1)
  _, s1, s2 = oracle.roco_forward(torch.zeros_like(q), k, v)
  inv = 1.0 / np.arange(1, S + 1)
  ref1 = np.cumsum(inv[::-1])[::-1]
  ref2 = np.cumsum((inv ** 2)[::-1])[::-1]
  assert np.abs(s1[0, 1].numpy() - ref1).max() < 1e-5
  assert np.abs(s2[0, 1].numpy() - ref2).max() < 1e-6
  out, s1, s2 = oracle.roco_forward(q, k, v)
  _, cs, cq, _ = brute.attention_stats(q, k, v)
  assert (s2 >= 0).all() and (s2 <= s1 + 1e-6).all()
  assert np.abs(s1.numpy() - cs).max() / cs.max() < 2e-3
  assert np.abs(s2.numpy() - cq).max() / cq.max() < 4e-3
  _, h2o = oracle.h2o_forward(q, k, v)
  assert torch.equal(h2o, s1)
  mean, var = oracle.roco_mean_var(s1, s2, S)
  assert torch.allclose(mean.sum(-1), torch.ones(1, 2), rtol=1e-5) and (var > -1e-7).all()


def test_keyformer_reductions_and_brute_force():
  S = 64
  q, k, v = _inputs(S=S, D=64, seed=2)
  _, h2o = oracle.h2o_forward(q, k, v)
  ones = torch.ones(1, 2, S, S)
  out, kf = oracle.keyformer_forward(q, k, v, ones, tau=1.0)
  # no noise, tau = 1: the perturbed softmax is the plain softmax
  assert torch.allclose(kf, h2o, rtol=1e-6, atol=1e-7)
  assert torch.equal(out, oracle.attn_forward(q, k, v))
  # tau -> inf: uniform over the visible keys, whatever the noise
  er = oracle.prepare_exp_rand(1, 2, S, S, seed=5)
  _, kf_inf = oracle.keyformer_forward(q, k, v, er, tau=1e9)
  harm = np.concatenate([[0.0], np.cumsum(1.0 / np.arange(1, S + 1))])
  assert np.abs(kf_inf[0, 0].numpy() - (harm[S] - harm[:S])).max() < 1e-4
  # random noise, reference default tau = 1.5, against fp64 brute force
  _, kf = oracle.keyformer_forward(q, k, v, er)
  _, _, _, ref = brute.attention_stats(q, k, v, exp_rand=er, tau=1.5)
  assert np.abs(kf.numpy() - ref).max() / ref.max() < 2e-3
  assert torch.allclose(kf.sum(-1), torch.full((1, 2), float(S)), rtol=1e-5)
  # sign of the Gumbel term: a huge exp_rand on one key column pushes its score down
  er2 = torch.ones(1, 2, S, S); er2[..., 3] = 1e4
  _, kf2 = oracle.keyformer_forward(q, k, v, er2, tau=1.0)
  assert (kf2[..., 3] < 1e-2 * h2o[..., 3]).all()


# ------------------------------------------------------------------ linear attention

def test_ea_closed_forms_and_brute_force():
  q, k, v = _inputs(B=2, S=48, H=2, D=64, seed=4)
  out = oracle.ea_forward(q, k, v)
  assert out.dtype == torch.float16 and out.shape == q.shape
  assert np.abs(out.float().numpy() - brute.ea(q, k, v)).max() < 2e-3
  # rows of Qs and columns of Ks sum to one: constant V passes through unchanged
  c = torch.full_like(v, 0.75)
  assert (oracle.ea_forward(q, k, c).float() - 0.75).abs().max() < 1e-3
  # Q = K = 0: uniform weights on both sides => every output row is the token mean of V
  z = torch.zeros_like(q)
  ref = v.float().mean(dim=1, keepdim=True).mean(dim=3, keepdim=True) * 0 + v.float().mean(dim=1, keepdim=True)
  got = oracle.ea_forward(z, z, v).float()
  # Qs uniform over D averages KV rows; Ks uniform over S makes every KV row the token mean of V
  assert (got - ref.expand_as(got)).abs().max() < 1e-3


def test_linear_cores_head_dim_32_brute_force():
  q, k, v = _inputs(B=1, S=33, H=3, D=32, seed=12)
  assert np.abs(oracle.ea_forward(q, k, v).float().numpy() - brute.ea(q, k, v)).max() < 2e-3
  ref = brute.sima(q, k, v)
  assert np.abs(oracle.sima_forward(q, k, v, out_dtype=torch.float32).numpy() - ref).max() / np.abs(ref).max() < 1e-5


def test_sima_invariants_and_brute_force():
  q, k, v = _inputs(B=1, S=40, H=2, D=64, seed=6)
  out32 = oracle.sima_forward(q, k, v, out_dtype=torch.float32)
  ref = brute.sima(q, k, v)
  assert np.abs(out32.numpy() - ref).max() / np.abs(ref).max() < 1e-5
  raw = oracle.sima_forward(q, k, v, normalize_q=False, out_dtype=torch.float32)
  ref_raw = brute.sima(q, k, v, normalize_q=False)
  assert np.abs(raw.numpy() - ref_raw).max() / np.abs(ref_raw).max() < 1e-5
  # positive rescaling of Q or K leaves the normalised form unchanged
  out_scaled = oracle.sima_forward(q * 2, k * 0.5, v, out_dtype=torch.float32)
  assert torch.allclose(out_scaled, out32, rtol=1e-5, atol=1e-9)
  # K >= 0 and constant V: Kh^T V = c for every channel => O[s,e] = c * sum_d Qh[s,d]
  kp = k.abs()
  c = torch.full_like(v, 0.5)
  got = oracle.sima_forward(q, kp, c, out_dtype=torch.float32)
  qh = q.transpose(1, 2).float(); qh = qh / qh.abs().sum(dim=2, keepdim=True)
  want = 0.5 * qh.sum(dim=3, keepdim=True).expand_as(qh).transpose(1, 2)
  assert torch.allclose(got, want, rtol=1e-4, atol=1e-8)


def test_linear_block_identity_bias_and_brute_force():
  B, S, H, D = 2, 24, 2, 64
  C = H * D
  x, w_qkv, b_qkv, w_out, b_out = oracle.prepare_block_inputs(B, S, H, D, seed=8)
  # fp64 index-form brute force; a transposed weight, a swapped q/k/v slot or a wrong head split fails it
  for fn, core, kw in ((oracle.ea_block_forward, brute.ea, {}), (oracle.sima_block_forward, brute.sima, {}),
                       (oracle.sima_block_forward, brute.sima, {"normalize_q": False})):
    got = fn(x, w_qkv, b_qkv, w_out, b_out, H, **kw).float().numpy()
    ref = brute.linear_block(core, x, w_qkv, b_qkv, w_out, b_out, H, **kw)
    assert np.abs(got - ref).max() <= 4e-3 * max(1.0, np.abs(ref).max()), (fn.__name__, kw)
  # stacked identities and zero biases: the block is the core on (x, x, x), bit for bit
  eye = torch.eye(C, dtype=torch.float16)
  z3, z1 = torch.zeros(3 * C, dtype=torch.float16), torch.zeros(C, dtype=torch.float16)
  x4 = x.reshape(B, S, H, D)
  assert torch.equal(oracle.ea_block_forward(x, torch.cat([eye, eye, eye]), z3, eye, z1, H),
                     oracle.ea_forward(x4, x4, x4).reshape(B, S, C))
  assert torch.equal(oracle.sima_block_forward(x, torch.cat([eye, eye, eye]), z3, eye, z1, H),
                     oracle.sima_forward(x4, x4, x4).reshape(B, S, C))
  # x = 0: q, k, v are their bias rows for every token; V constant over tokens passes through EA unchanged,
  # so y = w_out b_v + b_out (b_v = the third slot of the fused bias)
  y0 = oracle.ea_block_forward(torch.zeros_like(x), w_qkv, b_qkv, w_out, b_out, H).float()
  want = w_out.float() @ b_qkv[2 * C:].float() + b_out.float()
  assert (y0 - want).abs().max() < 2e-3


# ------------------------------------------------------------------ epilogues, recipes, chunking

def test_heavy_hitters_and_gap_rule():
  score = torch.tensor([[[0.1, 5.0, 3.0, 3.0000001, 0.2, 4.0, 0.0, 1.0]]])
  idx = oracle.heavy_hitters(score, 3)
  assert set(idx[0, 0].tolist()) in ({1, 5, 2}, {1, 5, 3})
  assert oracle.topk_agreement(idx, score, 3) == 0
  # swapping the near-tied pair is allowed, dropping a clear heavy hitter is not
  assert oracle.topk_agreement(torch.tensor([[[1, 5, 3]]]), score, 3) == 0
  assert oracle.topk_agreement(torch.tensor([[[1, 2, 3]]]), score, 3) == 1
  assert oracle.topk_agreement(torch.tensor([[[1, 5, 7]]]), score, 3) == 1


def test_chunked_over_heads_is_identical():
  q, k, v = _inputs(B=1, S=64, H=4, D=64, seed=9)
  full = oracle.roco_forward(q, k, v)
  part = oracle.chunked_over_heads(oracle.roco_forward, (q, k, v), head_chunk=1)
  for a, b in zip(full, part):
    assert torch.equal(a, b)
  er = oracle.prepare_exp_rand(1, 4, 64, 64)
  full = oracle.keyformer_forward(q, k, v, er, tau=1.0)
  part = oracle.chunked_over_heads(oracle.keyformer_forward, (q, k, v), head_chunk=2, extra=(er,), tau=1.0)
  for a, b in zip(full, part):
    assert torch.equal(a, b)


def test_prepare_inputs_is_seeded_and_ordered():
  q, k, v = oracle.prepare_inputs(1, 16, 2, 64, seed=0)
  g = torch.Generator().manual_seed(0)
  assert torch.equal(q, torch.randn(1, 16, 2, 64, dtype=torch.float16, generator=g))
  assert torch.equal(k, torch.randn(1, 16, 2, 64, dtype=torch.float16, generator=g))
  assert not torch.equal(q, oracle.prepare_inputs(1, 16, 2, 64, seed=1)[0])
  er = oracle.prepare_exp_rand(1, 2, 16, 16)
  assert (er >= 1).all() and er.dtype == torch.float32


def test_reference_rounding_points():
  # the eager definition rounds QK^T to fp16 and divides by sqrt(D) in fp16 before the fp32 softmax
  q, k, v = _inputs(S=64, D=128, seed=11)
  scores, probs = oracle.cases._masked_scores_probs(q, k)
  assert scores.dtype == torch.float16 and probs.dtype == torch.float32
  s32 = torch.matmul(q.transpose(1, 2).float(), k.transpose(1, 2).float().transpose(-2, -1))
  manual = (s32.half().float() / torch.tensor(math.sqrt(128), dtype=torch.float32)).half()
  tri = torch.tril(torch.ones(64, 64, dtype=torch.bool))
  assert torch.equal(scores[..., tri], manual[..., tri])
  assert torch.isinf(scores[..., ~tri]).all()


# ------------------------------------------------------------------ seeded noise stream

def test_noise_stream_statistics():
  E = oracle.seeded_exp_rand(1234, 1, 2, 256, 256)
  assert E.dtype == torch.float32 and (E > 0).all() and torch.isfinite(E).all()
  u = torch.exp(-E.double())
  # uniform(0,1): mean 1/2, var 1/12; Exp(1): mean 1, var 1
  assert abs(u.mean().item() - 0.5) < 5e-3 and abs(u.var().item() - 1 / 12) < 2e-3
  assert abs(E.mean().item() - 1.0) < 2e-2 and abs(E.var().item() - 1.0) < 5e-2
  # Kolmogorov-Smirnov against U(0,1)
  from scipy import stats
  assert stats.kstest(u[0, 0].flatten().numpy()[:20000], "uniform").pvalue > 1e-3
  # neighbouring rows / columns / heads are uncorrelated
  x = u[0, 0] - 0.5
  n = x.numel()
  for a, b in ((x[1:], x[:-1]), (x[:, 1:], x[:, :-1]), (x, u[0, 1] - 0.5)):
    corr = (a * b).mean().item() / (1 / 12)
    assert abs(corr) < 5 / math.sqrt(n)
  # a different seed gives a different stream; the same seed is reproducible
  assert not torch.equal(E, oracle.seeded_exp_rand(1235, 1, 2, 256, 256))
  assert torch.equal(E[:, :, 5:9], oracle.seeded_exp_rand(1234, 1, 2, 4, 256, row_offset=5))


def test_lowbias32_known_answers():
  # computed by hand-running the definition with Python integers (independent of numpy's wraparound)
  def ref(x):
    x &= 0xFFFFFFFF
    x ^= x >> 16; x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15; x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x
  xs = [0, 1, 2, 0xFFFFFFFF, 0x12345678, 0x9E3779B9]
  got = oracle.lowbias32(np.array(xs, dtype=np.uint64))
  assert [int(g) for g in got] == [ref(x) for x in xs]
  assert int(oracle.lowbias32(0)) == 0 and len(set(int(g) for g in got)) == len(xs)
  # the element combiner, by hand with Python integers: seed 7, head 3, row 11, column 5
  seed, bh, i, j = 7, 3, 11, 5
  k0 = ref((seed & 0xFFFFFFFF) ^ ref(bh + 0x9E3779B9)); k1 = ref((seed >> 32) ^ k0 ^ 0x85EBCA6B)
  a, b = ref(i ^ k0), ref(j ^ k1) | 1
  x = (a * b) & 0xFFFFFFFF; x ^= x >> 16
  assert int(oracle.noise_u32(seed, bh, [i], [j])[0, 0]) == x
  E = oracle.seeded_exp_rand(seed, 1, 4, 12, 6)[0, 3, 11, 5].item()
  assert abs(E - -math.log(((x >> 9) + 0.5) * 2.0 ** -23)) < 1e-6 * E


def test_noise_stream_has_no_lattice_structure():
  # sums and differences over 2x2 minors: u_ij - u_ij' - u_i'j + u_i'j' (mod 1) is uniform for independent
  # draws; a generator that only adds a row term and a column term before a weak mix fails this badly
  from scipy import stats
  x = oracle.noise_u32(99, 0, np.arange(768), np.arange(768))
  u = ((x >> np.uint32(9)).astype(np.float64) + 0.5) * 2.0 ** -23
  d = (u[:-1, :-1] - u[:-1, 1:] - u[1:, :-1] + u[1:, 1:] + 0.5) % 1.0
  assert stats.chisquare(np.bincount((d.flatten() * 256).astype(int) % 256, minlength=256)).pvalue > 1e-4
  pairs = np.bincount((u[:, :-1].flatten() * 64).astype(int) * 64 + (u[:, 1:].flatten() * 64).astype(int), minlength=4096)
  assert stats.chisquare(pairs).pvalue > 1e-4
  pairs = np.bincount((u[:-1].flatten() * 64).astype(int) * 64 + (u[1:].flatten() * 64).astype(int), minlength=4096)
  assert stats.chisquare(pairs).pvalue > 1e-4
  # the least significant bits that reach the uniform (bits 9..12 of the folded product; without the fold
  # x ^= x >> 16 they fail this: bit k of a product depends on bits 0..k of its factors only): balanced, and
  # independent between neighbours along either axis
  low = (x >> np.uint32(9)) & np.uint32(15)
  assert stats.chisquare(np.bincount(low.flatten(), minlength=16)).pvalue > 1e-4
  assert stats.chisquare(np.bincount((low[:, :-1] * 16 + low[:, 1:]).flatten(), minlength=256)).pvalue > 1e-4
  assert stats.chisquare(np.bincount((low[:-1] * 16 + low[1:]).flatten(), minlength=256)).pvalue > 1e-4


@pytest.mark.parametrize("seed", [1, 99, 2024, 123456789, 2 ** 40 + 7])
def test_noise_stream_over_seeds_and_heads_and_its_multiplicative_relation(seed):
  """The element word is a product a_i * b_j (mod 2^32) of a row and a column term, folded once.  Before the
  fold the words of every 2x2 minor satisfy x_ij x_kl == x_il x_kj (mod 2^32) exactly; the emitted words and the
  uniforms made of them must show nothing of it.  Checked for several seeds (one above 2^32) and (b, h) pairs."""
  from scipy import stats
  rng = np.random.default_rng(0)
  for bh in (0, 5, 31):
    x = oracle.noise_u32(seed, bh, np.arange(384), np.arange(384))
    u = ((x >> np.uint32(9)).astype(np.float64) + 0.5) * 2.0 ** -23
    assert stats.kstest(u.flatten()[::5], "uniform").pvalue > 1e-3
    # products of the emitted words over 2x2 minors: never equal, top bytes agree at the chance rate 1/256
    xa = (x[:-1, :-1].astype(np.uint64) * x[1:, 1:].astype(np.uint64)) & np.uint64(0xFFFFFFFF)
    xb = (x[:-1, 1:].astype(np.uint64) * x[1:, :-1].astype(np.uint64)) & np.uint64(0xFFFFFFFF)
    assert (xa == xb).mean() < 1e-4
    agree = ((xa >> np.uint64(24)) == (xb >> np.uint64(24))).mean()
    n = xa.size
    assert abs(agree - 1 / 256) < 5 * math.sqrt((1 / 256) * (255 / 256) / n)
    # the same relation in the domain the kernels use the numbers in: log u_ij + log u_kl - log u_il - log u_kj
    # has the distribution it has for independent uniforms
    L = np.log(u)
    d = (L[:-1, :-1] + L[1:, 1:] - L[:-1, 1:] - L[1:, :-1]).flatten()[::7]
    r = np.log(rng.random((4, d.size)))
    assert stats.ks_2samp(d, r[0] + r[1] - r[2] - r[3]).pvalue > 1e-3
    # different heads and different seeds do not share rows
    other = oracle.noise_u32(seed, bh + 1, np.arange(384), np.arange(384))
    assert (other == x).mean() < 1e-3
  assert not np.array_equal(oracle.noise_u32(seed, 0, np.arange(8), np.arange(8)), oracle.noise_u32(seed + 1, 0, np.arange(8), np.arange(8)))


# ------------------------------------------------------------------ SnapKV, CoRM, Gemma2

def test_snapkv_pool_closed_forms_and_brute_force():
  q, k, v = _inputs(S=48, H=2, D=64, seed=11)
  out_h, score_h = oracle.h2o_forward(q, k, v)
  out1, s1 = oracle.snapkv_forward(q, k, v, kernel_size=1)
  assert torch.equal(out1, out_h) and torch.equal(s1, score_h)           # a window of one is the identity
  out5, s5 = oracle.snapkv_forward(q, k, v)                               # reference default: 5
  assert torch.equal(out5, out_h) and s5.shape == score_h.shape
  _, cs, _, _ = brute.attention_stats(q, k, v)
  np.testing.assert_allclose(s5.numpy(), brute.avg_pool_same(cs, 5), rtol=2e-3, atol=1e-6)
  # edges: the first output averages only three real entries but still divides by five
  np.testing.assert_allclose(s5[..., 0].numpy(), (cs[..., 0] + cs[..., 1] + cs[..., 2]) / 5, rtol=2e-3)
  # q == 0: score_j = H_S - H_j, smooth, so interior windows sit between their neighbours' extremes
  z = torch.zeros_like(q)
  _, sz = oracle.snapkv_forward(z, k, v, kernel_size=3)
  _, hz = oracle.h2o_forward(z, k, v)
  mid = (hz[..., :-2] + hz[..., 1:-1] + hz[..., 2:]) / 3
  np.testing.assert_allclose(sz[..., 1:-1].numpy(), mid.numpy(), rtol=1e-5)


def test_corm_closed_forms_and_brute_force():
  S = 40
  q, k, v = _inputs(S=S, H=2, D=64, seed=12)
  rule = oracle.corm_mask_rule(S, S)
  assert rule.shape == (S, S) and rule[0, 0] == 1.0 and rule[9, 3] == np.float32(1.0) / np.float32(10.0)
  out, keep = oracle.corm_forward(q, k, v, rule)
  assert keep.dtype == torch.bool and keep.shape == (1, 2, S)
  assert torch.equal(out, oracle.attn_forward(q, k, v))
  assert keep[..., 0].all()                                               # p_00 == 1 >= 1
  # q == 0: every visible probability equals 1/(i+1) exactly, so every key is kept
  _, keep0 = oracle.corm_forward(torch.zeros_like(q), k, v, rule)
  assert keep0.all()
  # an all-ones threshold keeps only keys that some row attends to with probability one: key 0 (row 0)
  ones = torch.ones(S, S)
  _, keep1 = oracle.corm_forward(q, k, v, ones)
  assert keep1[..., 0].all() and not keep1[..., 1:].any()
  # fp64 brute force wherever the decision is not within 1e-3 of the boundary
  ratio = brute.corm_ratio(q, k, rule)
  clear = np.abs(ratio - 1.0) > 1e-3
  assert clear.mean() > 0.9
  assert np.array_equal(keep.numpy()[clear], (ratio >= 1.0)[clear])
  assert 0.05 < keep.float().mean().item() < 0.999                         # the test exercises both outcomes
  m = oracle.corm_margin(q, k, rule)
  np.testing.assert_allclose(m.numpy(), ratio, rtol=3e-3)
  assert torch.equal(m >= 1, keep) or (np.abs(m.numpy() - 1) < 1e-6).any()


def test_gemma2_softcap_limits_and_brute_force():
  q, k, v = _inputs(S=48, H=2, D=64, seed=13)
  # a large power-of-two cap: logit / cap is exact unless it falls into fp16 subnormals (|logit| < 0.03),
  # tanh(y) == y in fp16 for |y| < 0.027, times cap is exact -> plain attention up to a few last-bit flips
  big = oracle.gemma2_forward(q, k, v, softcap=512.0)
  plain = oracle.attn_forward(q, k, v)
  assert (big.float() - plain.float()).abs().max().item() <= 2e-3
  assert (big == plain).float().mean().item() > 0.99
  # a tiny cap squashes every logit to (-cap, cap): probabilities ~ uniform over the visible prefix
  o_small = oracle.gemma2_forward(q, k, v, softcap=1e-3)
  prefix = torch.cumsum(v.float(), dim=1) / torch.arange(1, 49).view(1, -1, 1, 1)
  assert (o_small.float() - prefix).abs().max().item() < 5e-3
  ref = brute.softcap_attention(q, k, v, 50.0)
  assert np.abs(oracle.gemma2_forward(q, k, v).float().numpy() - ref).max() < 4e-3
  # the cap matters: with cap 2 the result differs clearly from plain attention and matches the brute force
  ref2 = brute.softcap_attention(q, k, v, 2.0)
  o2 = oracle.gemma2_forward(q, k, v, softcap=2.0).float().numpy()
  assert np.abs(o2 - ref2).max() < 4e-3
  assert np.abs(o2 - oracle.attn_forward(q, k, v).float().numpy()).max() > 2e-2


# ------------------------------------------------------------------ 2-D harness form, grouped queries

def test_attn2d_and_grouped_h2o_against_expanded_heads_and_brute_force():
  S, H, D = 40, 4, 64
  q, k, v = _inputs(S=S, H=H, D=D, seed=14)
  q2, k2, v2 = (t[0].reshape(S, H * D) for t in (q, k, v))
  # one k/v head per query head: the 4-D cases on the same data, bit for bit
  assert torch.equal(oracle.attn2d_forward(q2, k2, v2, H, H, D), oracle.attn_forward(q, k, v)[0].reshape(S, H * D))
  o2, s2 = oracle.attn_h2o2d_forward(q2, k2, v2, H, H, D)
  oh, sh = oracle.h2o_forward(q, k, v)
  assert torch.equal(o2, oh[0].reshape(S, H * D)) and torch.equal(s2, sh[0])
  # grouped: 4 query heads on 2 k/v heads == the ungrouped case on repeated k/v heads, scores averaged per pair
  Hkv = 2
  kg, vg = k[:, :, :Hkv].contiguous(), v[:, :, :Hkv].contiguous()
  kr, vr = kg.repeat_interleave(H // Hkv, dim=2), vg.repeat_interleave(H // Hkv, dim=2)
  og, sg = oracle.attn_h2o2d_forward(q2, kg[0].reshape(S, Hkv * D), vg[0].reshape(S, Hkv * D), Hkv, H, D)
  orf, srf = oracle.h2o_forward(q, kr, vr)
  assert torch.equal(og, orf[0].reshape(S, H * D))
  assert torch.allclose(sg, srf[0].view(Hkv, H // Hkv, S).mean(dim=1), rtol=1e-6)
  assert abs(sg.sum().item() - Hkv * S) < 1e-3 * S                         # every averaged row still sums to one
  # independent fp64 definition with explicit head // group indexing
  O, cs, _, _ = brute.attention_stats(q, kr, vr)
  np.testing.assert_allclose(sg.numpy(), cs[0].reshape(Hkv, H // Hkv, S).mean(axis=1), rtol=2e-3)
  assert np.abs(og.float().numpy() - O[0].reshape(S, H * D)).max() < 4e-3
  # query head 1 must read k/v head 0, not 1: swapping the two k/v heads changes its output
  ksw = kg[:, :, [1, 0]].contiguous()
  osw = oracle.attn2d_forward(q2, ksw[0].reshape(S, Hkv * D), vg[0].reshape(S, Hkv * D), Hkv, H, D)
  assert (osw.view(S, H, D)[:, 1] - og.view(S, H, D)[:, 1]).abs().max().item() > 1e-2
  # unmasked variant: every key is visible to every row
  of, sf = oracle.attn_h2o2d_forward(q2, k2, v2, H, H, D, masked=False)
  assert abs(sf.sum().item() - H * S) < 1e-3 * S and (sf[:, -1] > 0.1).all()


# ------------------------------------------------------------------ RoCo mean / variance epilogue, harness metrics

def _mean_var_impls():
  from flashtensor_amd import kernels
  return [("oracle", oracle.roco_mean_var), ("product", kernels.RoCo.mean_var)]


@pytest.mark.parametrize("which", [0, 1])
def test_roco_mean_var_zero_q_closed_form(which):
  """q == 0: p_ij = 1/(i+1) for j <= i, else 0.  Over the S query rows key j then has
  mean_j = (H_S - H_j) / S and population variance sum_{i>=j} (i+1)^-2 / S - mean_j^2; a variance that
  forgets mean^2, divides by S - 1, or takes the mean over the visible rows only fails."""
  name, fn = _mean_var_impls()[which]
  S = 80
  q, k, v = _inputs(S=S, D=64, seed=1)
  _, s1, s2 = oracle.roco_forward(torch.zeros_like(q), k, v)
  mean, var = fn(s1, s2, S)
  inv = 1.0 / np.arange(1, S + 1)
  ref_mean = np.cumsum(inv[::-1])[::-1] / S
  ref_var = np.cumsum((inv ** 2)[::-1])[::-1] / S - ref_mean ** 2
  assert np.abs(mean[0, 0].numpy() - ref_mean).max() < 1e-7, name
  assert np.abs(var[0, 1].numpy() - ref_var).max() < 1e-7, name
  # the wrong formulas are far outside that bar
  assert np.abs(np.cumsum((inv ** 2)[::-1])[::-1] / S - ref_var).max() > 1e-3
  assert np.abs((ref_var * S / (S - 1)) - ref_var).max() > 1e-5


@pytest.mark.parametrize("which", [0, 1])
@pytest.mark.parametrize("S,Skv", [(48, 48), (24, 56)])
def test_roco_mean_var_against_numpy_on_brute_force_probs(which, S, Skv):
  """mean / var over the query axis of the fp64 masked probability matrix (masked pairs are zeros, as in
  probs.mean(2) / probs.var(2, unbiased=False) of the eager tensors of cases/kernels/roco.py:42-46)."""
  name, fn = _mean_var_impls()[which]
  q, k, v = _inputs(B=1, S=S, H=2, D=64, seed=9, kv_len=Skv)
  _, s1, s2 = oracle.roco_forward(q, k, v)
  mean, var = fn(s1, s2, S)
  for h in range(2):
    _, p = brute._probs(q.numpy(), k.numpy(), 0, h)
    assert p.shape == (S, Skv)
    np.testing.assert_allclose(mean[0, h].numpy(), p.mean(axis=0), rtol=2e-3, atol=1e-7, err_msg=name)
    np.testing.assert_allclose(var[0, h].numpy(), p.var(axis=0), rtol=6e-3, atol=1e-7, err_msg=name)


def _loss_impls():
  from flashtensor_amd import utils
  from oracle import metrics
  return [("oracle", metrics.loss), ("product", utils.loss)]


@pytest.mark.parametrize("which", [0, 1])
def test_loss_known_answers(which):
  """python/asuka/utils.py:61-76 by hand: |d| = [0.5, 0, 1, 2], |ref| = [1, 2, 4, 0]."""
  name, loss = _loss_impls()[which]
  out = torch.tensor([[1.5, 2.0], [-3.0, 2.0]], dtype=torch.float16)
  ref = torch.tensor([[1.0, 2.0], [-4.0, 0.0]], dtype=torch.float16)
  r = loss(out, ref, remove_zero=True)       # the zero denominator becomes 1: rel = [0.5, 0, 0.25, 2]
  assert r["remove_zero"] is True
  assert r["abs_max"] == 2.0 and r["abs_mean"] == pytest.approx(0.875)
  assert r["rel_max"] == 2.0 and r["rel_mean"] == pytest.approx(0.6875)
  r = loss(out, ref)                          # kept: 2 / 0 = inf
  assert r["remove_zero"] is False and r["abs_max"] == 2.0 and math.isinf(r["rel_max"]) and math.isinf(r["rel_mean"])
  r = loss(out[:1], ref[:1])                  # no zero in the reference: rel = [0.5, 0]
  assert r["rel_max"] == 0.5 and r["rel_mean"] == 0.25 and r["abs_mean"] == 0.25
  assert not ref[1, 1].item() and ref.dtype == torch.float16   # the inputs are left as they were
  # integer tensors: mismatch count and fraction
  for dt in (torch.int32, torch.int64):
    a = torch.tensor([1, 2, 3, 4, 5], dtype=dt)
    b = torch.tensor([1, 0, 3, 0, 5], dtype=dt)
    assert loss(a, b) == {"err_num": 2, "err": 0.4}, name
  with pytest.raises(AssertionError):
    loss(torch.zeros(2, 3), torch.zeros(3, 2))


def test_one_fp16_ulp_of_a_tie_logit_exceeds_the_score_bar():
  """Why the GPU parity tests carry an allowance for rounding ties.  Seed 151029 (found by a random sweep): the
  exact QK^T of query 191 and key 313 of head (0, 0) is 20.8671875 + 5.5e-7, a hair from the midpoint of the fp16
  neighbours 20.859375 and 20.875, so the order of the fp32 accumulation decides which one the reference's fp16
  QK^T holds; that row carries 93 % of the key's KeyFormer score at tau = 0.5, and the two valid roundings give
  scores 3.6e-3 apart, more than the 1e-3 bar.  Deterministic: both roundings are built here by hand."""
  B, S, kv, H, D, seed, (b, h, i, j), tau = 2, 246, 408, 2, 64, 151029, (0, 0, 191, 313), 0.5
  q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed, kv_len=kv)
  exact = float(q[b, i, h].double() @ k[b, j, h].double())
  lo, hi = np.float16(20.859375), np.float16(20.875)
  assert abs(exact - (float(lo) + float(hi)) / 2) < 1e-4 * float(hi - lo)
  es = oracle.seeded_exp_rand(seed, B, H, S, kv)[b, h]
  raw = (q[b, :, h].double() @ k[b, :, h].double().T).half()                   # exact sums rounded once
  mask = torch.triu(torch.full((S, kv), float("-inf")), diagonal=kv - S + 1)
  scores = []
  for value in (lo, hi):
    r = raw.clone()
    r[i, j] = float(value)
    z = ((r / math.sqrt(D)).float() + mask - es.log()) / tau
    scores.append(torch.softmax(z, -1).sum(0)[j].item())
  assert abs(scores[0] - scores[1]) / scores[1] > 3e-3
  # and the allowance the GPU tests compute for this key covers it, while most keys get none
  sc = ((raw / math.sqrt(D)).float() + mask)[None, None]
  w = torch.softmax((sc - es.log()) / tau, -1)
  slack = brute.rounding_tie_slack(q[b:b + 1, :, h:h + 1], k[b:b + 1, :, h:h + 1], w, tau=tau)
  assert slack[0, 0, j] > 3e-3 and (slack > 2.5e-4).mean() < 0.02
