"""The CPU oracle against the committed golden vectors (tests/golden/*.npz, written by make_golden.py)."""
import glob
import os

import numpy as np
import pytest
import torch

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(path):
  z = np.load(path, allow_pickle=False)
  return {k: z[k] for k in z.files}


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "softmax_*.npz"))), ids=os.path.basename)
def test_softmax_cases_match_golden(path):
  g = _load(path)
  B, S, H, D, seed = (int(g[k]) for k in ("B", "S", "H", "D", "seed"))
  q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
  out, s1, s2 = oracle.roco_forward(q, k, v)
  # thread count may change the reduction order of the CPU GEMM / sums by an ulp
  assert np.abs(out.float().numpy() - g["out"].astype(np.float32)).max() <= 2e-3
  np.testing.assert_allclose(s1.numpy(), g["colsum"], rtol=1e-5, atol=1e-7)
  np.testing.assert_allclose(s2.numpy(), g["colsumsq"], rtol=1e-5, atol=1e-8)
  _, kf = oracle.keyformer_forward(q, k, v, oracle.prepare_exp_rand(B, H, S, S, seed=seed), tau=1.5)
  np.testing.assert_allclose(kf.numpy(), g["kf_tensor_tau15"], rtol=1e-5, atol=1e-7)
  _, kfs = oracle.keyformer_forward(q, k, v, oracle.seeded_exp_rand(int(g["kf_seed"]), B, H, S, S), tau=1.0)
  np.testing.assert_allclose(kfs.numpy(), g["kf_seeded_tau1"], rtol=1e-5, atol=1e-7)
  assert oracle.topk_agreement(torch.from_numpy(g["topk"]), s1, S // 8) == 0


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "linear_*.npz"))), ids=os.path.basename)
def test_linear_cases_match_golden(path):
  g = _load(path)
  B, S, H, D, seed = (int(g[k]) for k in ("B", "S", "H", "D", "seed"))
  q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
  assert np.abs(oracle.ea_forward(q, k, v).float().numpy() - g["ea"].astype(np.float32)).max() <= 1e-3
  np.testing.assert_allclose(oracle.sima_forward(q, k, v, out_dtype=torch.float32).numpy(), g["sima"], rtol=1e-4, atol=1e-9)
  np.testing.assert_allclose(oracle.sima_forward(q, k, v, normalize_q=False, out_dtype=torch.float32).numpy(),
                             g["sima_rawq"], rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "next_*.npz"))), ids=os.path.basename)
def test_next_cases_match_golden(path):
  g = _load(path)
  B, S, H, D, seed = (int(g[k]) for k in ("B", "S", "H", "D", "seed"))
  q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
  rule = oracle.corm_mask_rule(S, S)
  np.testing.assert_allclose(oracle.snapkv_forward(q, k, v)[1].numpy(), g["snapkv5"], rtol=1e-5, atol=1e-7)
  ratio = oracle.corm_margin(q, k, rule).numpy()
  np.testing.assert_allclose(ratio, g["corm_ratio"], rtol=1e-5)
  clear = np.abs(g["corm_ratio"] - 1) > 1e-4
  assert np.array_equal(oracle.corm_forward(q, k, v, rule)[1].numpy()[clear], g["corm_keep"][clear])
  assert np.abs(oracle.gemma2_forward(q, k, v).float().numpy() - g["gemma2_cap50"].astype(np.float32)).max() <= 2e-3
  assert np.abs(oracle.gemma2_forward(q, k, v, softcap=2.0).float().numpy() - g["gemma2_cap2"].astype(np.float32)).max() <= 2e-3
  kg, vg = k[:, :, : H // 2].contiguous(), v[:, :, : H // 2].contiguous()
  og, sg = oracle.attn_h2o2d_forward(q[0].reshape(S, H * D), kg[0].reshape(S, H // 2 * D), vg[0].reshape(S, H // 2 * D), H // 2, H, D)
  assert np.abs(og.float().numpy() - g["gqa_out"].astype(np.float32)).max() <= 2e-3
  np.testing.assert_allclose(sg.numpy(), g["gqa_score"], rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "block_*.npz"))), ids=os.path.basename)
def test_block_cases_match_golden(path):
  g = _load(path)
  B, S, H, D, seed = (int(g[k]) for k in ("B", "S", "H", "D", "seed"))
  args = oracle.prepare_block_inputs(B, S, H, D, seed=seed)
  assert np.abs(oracle.ea_block_forward(*args, H).float().numpy() - g["ea_block"].astype(np.float32)).max() <= 2e-3
  assert np.abs(oracle.sima_block_forward(*args, H, normalize_q=False).float().numpy()
                - g["sima_block_rawq"].astype(np.float32)).max() <= 2e-3
  q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
  assert np.abs(oracle.ea_forward(q, k, v).float().numpy() - g["ea_core"].astype(np.float32)).max() <= 1e-3
  np.testing.assert_allclose(oracle.sima_forward(q, k, v, out_dtype=torch.float32).numpy(), g["sima_core"], rtol=1e-4, atol=1e-9)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "lindtype_*.npz"))), ids=os.path.basename)
def test_linear_cases_in_bf16_and_fp32_match_golden(path):
  g = _load(path)
  B, S, H, D, seed = (int(g[k]) for k in ("B", "S", "H", "D", "seed"))
  for tag, dt, tol in (("bf16", torch.bfloat16, 8e-3), ("f32", torch.float32, 1e-5)):
    q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed, dtype=dt)
    args = oracle.prepare_block_inputs(B, S, H, D, seed=seed, dtype=dt)
    assert np.abs(oracle.ea_forward(q, k, v).float().numpy() - g[f"ea_{tag}"]).max() <= tol
    np.testing.assert_allclose(oracle.sima_forward(q, k, v, out_dtype=torch.float32).numpy(), g[f"sima_{tag}_f32out"], rtol=1e-4, atol=1e-9)
    assert np.abs(oracle.ea_block_forward(*args, H).float().numpy() - g[f"ea_block_{tag}"]).max() <= 2 * tol
    assert np.abs(oracle.sima_block_forward(*args, H, normalize_q=False).float().numpy() - g[f"sima_block_rawq_{tag}"]).max() <= 2 * tol


def test_golden_files_present():
  assert len(glob.glob(os.path.join(GOLDEN, "*.npz"))) == 10
