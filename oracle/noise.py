"""Host twin of the counter-based noise generator used by the seeded KeyFormer mode.

TEST INFRASTRUCTURE (see `oracle/__init__.py`).  Integer arithmetic in numpy, bit-exact with the
device generator in `flashtensor_amd/csrc/noise.h`.

The reference has no in-kernel generator: its KeyFormer case takes the noise as an input tensor
`exp_rand[B,H,Sq,Skv]` (`cases/kernels/kf.py:19,36-37,48`) and only its stale MLIR snapshot names a
seeded source (`bench/keyformer.mlir:4,17`, `asuka.rng UNIT_GUMBEL`).  The seeded mode therefore
defines its own stream, and this module materialises exactly the tensor the kernel draws so that
`keyformer_forward(q, k, v, seeded_exp_rand(...), tau)` is the oracle for it.

Stream definition (all arithmetic mod 2**32):
    lowbias32(x): x ^= x>>16; x *= 0x7feb352d; x ^= x>>15; x *= 0x846ca68b; x ^= x>>16
    k0 = lowbias32(seed_lo ^ lowbias32(bh + 0x9E3779B9));  k1 = lowbias32(seed_hi ^ k0 ^ 0x85EBCA6B)
    a_i = lowbias32(i ^ k0);  b_j = lowbias32(j ^ k1) | 1;  x_ij = a_i * b_j;  x_ij ^= x_ij >> 16
    u_ij = ((x_ij >> 9) + 0.5) * 2**-23        in (0,1), exact in fp32
    E_ij = -ln(u_ij)                            ~ Exp(1);  g_ij = -ln(E_ij) ~ Gumbel(0,1)
with bh = b*H + h, i the query row and j the key column.
"""
import numpy as np

_M = np.uint64(0xFFFFFFFF)


def lowbias32(x):
  """32-bit integer finaliser (two multiply / xor-shift rounds); x: uint32 array or int."""
  x = np.asarray(x, dtype=np.uint64) & _M
  x ^= x >> np.uint64(16)
  x = (x * np.uint64(0x7FEB352D)) & _M
  x ^= x >> np.uint64(15)
  x = (x * np.uint64(0x846CA68B)) & _M
  x ^= x >> np.uint64(16)
  return x.astype(np.uint32)


def _keys(seed, bh):
  seed = int(seed) & 0xFFFFFFFFFFFFFFFF
  seed_lo, seed_hi = seed & 0xFFFFFFFF, seed >> 32
  bh = np.asarray(bh, dtype=np.uint64)
  k0 = lowbias32(np.uint64(seed_lo) ^ lowbias32((bh + np.uint64(0x9E3779B9)) & _M).astype(np.uint64))
  k1 = lowbias32(np.uint64(seed_hi) ^ k0.astype(np.uint64) ^ np.uint64(0x85EBCA6B))
  return k0, k1


def noise_u32(seed, bh, rows, cols):
  """x_ij for one (b,h) pair: rows, cols are 1-D integer arrays -> uint32 [len(rows), len(cols)]."""
  k0, k1 = _keys(seed, bh)
  a = lowbias32(np.asarray(rows, dtype=np.uint64) ^ k0.astype(np.uint64)).astype(np.uint64)
  b = lowbias32(np.asarray(cols, dtype=np.uint64) ^ k1.astype(np.uint64)).astype(np.uint64) | np.uint64(1)
  x = (a[:, None] * b[None, :]) & _M
  x ^= x >> np.uint64(16)
  return x.astype(np.uint32)


def seeded_exp_rand(seed, B, H, Sq, Skv, row_offset=0):
  """The fp32 tensor E[B,H,Sq,Skv] the seeded KeyFormer kernel draws (returned as a torch tensor)."""
  import torch
  out = np.empty((B, H, Sq, Skv), dtype=np.float32)
  rows = np.arange(row_offset, row_offset + Sq)
  cols = np.arange(Skv)
  for b in range(B):
    for h in range(H):
      x = noise_u32(seed, b * H + h, rows, cols)
      u = ((x >> np.uint32(9)).astype(np.float64) + 0.5) * 2.0 ** -23
      out[b, h] = (-np.log(u)).astype(np.float32)
  return torch.from_numpy(out)


def seeded_exp_rand_pairs(seed, H_total, pairs, Sq, Skv):
  """E for chosen (b, h) pairs of a problem with H_total heads, stacked as [1, len(pairs), Sq, Skv]: what
  `seeded_exp_rand(seed, B, H_total, Sq, Skv)[b, h]` holds for each pair, without the other heads."""
  import torch
  out = np.empty((1, len(pairs), Sq, Skv), dtype=np.float32)
  rows, cols = np.arange(Sq), np.arange(Skv)
  for n, (b, h) in enumerate(pairs):
    x = noise_u32(seed, b * H_total + h, rows, cols)
    u = ((x >> np.uint32(9)).astype(np.float64) + 0.5) * 2.0 ** -23
    out[0, n] = (-np.log(u)).astype(np.float32)
  return torch.from_numpy(out)
