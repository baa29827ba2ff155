"""Writes the golden vectors of tests/golden/*.npz from the CPU oracle.

    python tests/golden/make_golden.py

The reference ships no fixtures for this path, so these are regression vectors of the pinned oracle
(tests/test_oracle_pins.py): inputs are regenerated from the seed by oracle.prepare_inputs and are not
stored; the files hold the expected outputs only (fp16 O, fp32 scores, top-k indices).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# (name, B, S, H, D, seed)
SHAPES = [("s128_d128", 1, 128, 2, 128, 0), ("s256_d64", 1, 256, 2, 64, 0), ("s200_d128", 1, 200, 2, 128, 1)]
LIN_SHAPES = [("s256_d64", 1, 256, 2, 64, 0), ("s200_d64", 2, 200, 2, 64, 1)]
NEXT_SHAPES = [("s128_d128", 1, 128, 2, 128, 3), ("s200_d64", 1, 200, 4, 64, 4)]
BLOCK_SHAPES = [("s200_h2_d64", 2, 200, 2, 64, 5), ("s150_h4_d32", 1, 150, 4, 32, 6)]  # the second: head_dim 32, the .mlir's own
# the linear cores and blocks in the other two types they take: bf16 (the harness's switch) and fp32 (the .mlir's own)
DTYPE_SHAPES = [("s200_d64", 1, 200, 2, 64, 7)]
KF_SEED = 1234


def main():
  torch.set_num_threads(1)  # fixed reduction order
  for name, B, S, H, D, seed in SHAPES:
    q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
    out, s1, s2 = oracle.roco_forward(q, k, v)
    er = oracle.prepare_exp_rand(B, H, S, S, seed=seed)
    _, kf_t = oracle.keyformer_forward(q, k, v, er, tau=1.5)
    _, kf_s = oracle.keyformer_forward(q, k, v, oracle.seeded_exp_rand(KF_SEED, B, H, S, S), tau=1.0)
    np.savez_compressed(os.path.join(HERE, f"softmax_{name}.npz"), B=B, S=S, H=H, D=D, seed=seed, kf_seed=KF_SEED,
                        out=out.numpy(), colsum=s1.numpy(), colsumsq=s2.numpy(), kf_tensor_tau15=kf_t.numpy(),
                        kf_seeded_tau1=kf_s.numpy(), topk=oracle.heavy_hitters(s1, S // 8).numpy())
  for name, B, S, H, D, seed in LIN_SHAPES:
    q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
    np.savez_compressed(os.path.join(HERE, f"linear_{name}.npz"), B=B, S=S, H=H, D=D, seed=seed,
                        ea=oracle.ea_forward(q, k, v).numpy(),
                        sima=oracle.sima_forward(q, k, v, out_dtype=torch.float32).numpy(),
                        sima_rawq=oracle.sima_forward(q, k, v, normalize_q=False, out_dtype=torch.float32).numpy())
  for name, B, S, H, D, seed in NEXT_SHAPES:
    q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
    rule = oracle.corm_mask_rule(S, S)
    kg, vg = k[:, :, : H // 2].contiguous(), v[:, :, : H // 2].contiguous()  # grouped queries: two query heads per k/v head
    og, sg = oracle.attn_h2o2d_forward(q[0].reshape(S, H * D), kg[0].reshape(S, H // 2 * D), vg[0].reshape(S, H // 2 * D),
                                       H // 2, H, D)
    np.savez_compressed(os.path.join(HERE, f"next_{name}.npz"), B=B, S=S, H=H, D=D, seed=seed,
                        snapkv5=oracle.snapkv_forward(q, k, v)[1].numpy(),
                        corm_keep=oracle.corm_forward(q, k, v, rule)[1].numpy(),
                        corm_ratio=oracle.corm_margin(q, k, rule).numpy(),
                        gemma2_cap50=oracle.gemma2_forward(q, k, v).numpy(),
                        gemma2_cap2=oracle.gemma2_forward(q, k, v, softcap=2.0).numpy(),
                        gqa_out=og.numpy(), gqa_score=sg.numpy())
  for name, B, S, H, D, seed in BLOCK_SHAPES:
    args = oracle.prepare_block_inputs(B, S, H, D, seed=seed)
    q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed)
    np.savez_compressed(os.path.join(HERE, f"block_{name}.npz"), B=B, S=S, H=H, D=D, seed=seed,
                        ea_block=oracle.ea_block_forward(*args, H).numpy(),
                        sima_block_rawq=oracle.sima_block_forward(*args, H, normalize_q=False).numpy(),
                        ea_core=oracle.ea_forward(q, k, v).numpy(),
                        sima_core=oracle.sima_forward(q, k, v, out_dtype=torch.float32).numpy())
  for name, B, S, H, D, seed in DTYPE_SHAPES:
    arrays = {}
    for tag, dt in (("bf16", torch.bfloat16), ("f32", torch.float32)):
      q, k, v = oracle.prepare_inputs(B, S, H, D, seed=seed, dtype=dt)
      args = oracle.prepare_block_inputs(B, S, H, D, seed=seed, dtype=dt)
      # numpy has no bf16: every result is stored as fp32 (a bf16 value is exactly representable)
      arrays[f"ea_{tag}"] = oracle.ea_forward(q, k, v).float().numpy()
      arrays[f"sima_{tag}_f32out"] = oracle.sima_forward(q, k, v, out_dtype=torch.float32).numpy()
      arrays[f"ea_block_{tag}"] = oracle.ea_block_forward(*args, H).float().numpy()
      arrays[f"sima_block_rawq_{tag}"] = oracle.sima_block_forward(*args, H, normalize_q=False).float().numpy()
    np.savez_compressed(os.path.join(HERE, f"lindtype_{name}.npz"), B=B, S=S, H=H, D=D, seed=seed, **arrays)
  print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
  main()
