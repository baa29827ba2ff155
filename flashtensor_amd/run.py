"""Command-line harness in the manner of the reference's case scripts (cases/run.py:37-46 `-m <case>`,
cases/attn_h2o.py:84-164 shape options and the perf printout):

    python -m flashtensor_amd.run -m h2o [--batch_size 1] [--q_len 4096] [--kv_len 4096] [--type f16]
    python -m flashtensor_amd.run -m attn_h2o_2d --head_num 32 --kv_head_num 8 [--masked 1]

builds the case's callable through HipBuilder (or the 2-D harness classes), runs it on seeded N(0,1)
inputs and prints the timing line of `perf` with algorithmic GFLOP/s and GB/s.

    python -m flashtensor_amd.run -m h2o --check tests/golden/softmax_s128_d128.npz

additionally prints the harness's `loss(out, ref, remove_zero=True)` lines (cases/attn_h2o.py:144-145) against
expected outputs stored in an .npz: the file names the shape and the seed (B, S, H, D, seed), the inputs are
q, k, v ~ N(0,1) in that order from the CPU generator seeded with it (the recipe of cases/attn.py:89,99-101),
and the arrays listed in CHECK_KEYS are the expected results.  Where those come from is the file's business;
nothing here computes a CPU definition.
"""
import argparse

import numpy as np
import torch

from . import kernels, ops
from .builder import HipBuilder
from .utils import loss, perf

# expected-output arrays of a --check file, in the order of the case's results (None: no expectation stored)
CHECK_KEYS = {"attn": ["out"], "h2o": ["out", "colsum"], "roco": ["out", "colsum", "colsumsq"], "snapkv": [None, "snapkv5"],
              "gemma2": ["gemma2_cap50"], "ea": ["ea"], "sima": ["sima"]}

CASES_2D = {"attn_2d": kernels.Attn2D, "attn_h2o_2d": kernels.AttnH2O2D}


def build(args, device):
  """Returns (callable, input tensors, algorithmic GFLOP, algorithmic GB) for the parsed options."""
  dtype = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[args.type]
  torch.manual_seed(0)
  esz = 2
  if args.model_name in CASES_2D:
    model = CASES_2D[args.model_name](args.kv_head_num, args.head_num, args.head_dim, bool(args.masked))
    q = torch.randn(args.q_len, args.head_num * args.head_dim, dtype=dtype, device=device)
    k = torch.randn(args.kv_len, args.kv_head_num * args.head_dim, dtype=dtype, device=device)
    v = torch.randn(args.kv_len, args.kv_head_num * args.head_dim, dtype=dtype, device=device)
    pairs = args.q_len * args.kv_len * (0.5 if args.masked else 1.0)
    gflop = 4.0 * args.head_num * pairs * args.head_dim / 1e9
    gb = (2 * q.numel() + k.numel() + v.numel()) * esz / 1e9
    return model.forward, [q, k, v], gflop, gb
  hyper = {}
  linear = args.model_name in ("ea", "sima", "ea_block", "sima_block")
  block = args.model_name.endswith("_block")
  if linear:
    head_num, head_dim = args.head_num or 16, args.head_dim or 64
  else:
    head_num, head_dim = args.head_num or 32, args.head_dim or 128
  hyper.update(head_num=head_num, head_dim=head_dim)
  if not block:
    hyper.update(kv_head_num=head_num)
  f = HipBuilder(args.model_name, **hyper).build_callable()
  model = kernels.get_model(args.model_name, **hyper)
  inout = model.prepare(batch_size=args.batch_size, q_len=args.q_len, kv_len=args.kv_len, dtype=dtype, device=device)
  inputs = list(inout["input"].values())
  B, S, Skv = args.batch_size, args.q_len, args.kv_len
  if linear:
    gflop = 4.0 * B * head_num * S * head_dim * head_dim / 1e9
    if block:  # + the q/k/v and output projections, 2 M (3 C C + C C)
      gflop += 8.0 * B * S * (head_num * head_dim) ** 2 / 1e9
  else:
    gflop = 2.0 * B * head_num * S * Skv * head_dim / 1e9  # two causal contractions
  gb = 4.0 * B * S * head_num * head_dim * esz / 1e9
  return f, inputs, gflop, gb


def parse_args(argv=None):
  ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
  ap.add_argument("--model_name", "-m", default="h2o", choices=sorted(kernels.CASES) + sorted(CASES_2D))
  ap.add_argument("--batch_size", type=int, default=1)
  ap.add_argument("--q_len", type=int, default=4096)
  ap.add_argument("--kv_len", type=int, default=4096)
  ap.add_argument("--head_num", type=int, default=0)
  ap.add_argument("--kv_head_num", type=int, default=0)
  ap.add_argument("--head_dim", type=int, default=0)
  ap.add_argument("--masked", type=int, default=1)
  ap.add_argument("--type", default="f16", choices=["f16", "bf16", "f32"], help="f32: the linear cases only (the type of bench/ea.mlir)")
  ap.add_argument("--run", type=int, default=10)
  ap.add_argument("--warmup", type=int, default=10)
  ap.add_argument("--show_result", action="store_true")
  ap.add_argument("--check", default=None, metavar="FILE.npz",
                  help="expected outputs (and B, S, H, D, seed of the inputs) for the loss lines; cases: " + " ".join(sorted(CHECK_KEYS)))
  args = ap.parse_args(argv)
  if args.model_name in CASES_2D:
    args.head_num = args.head_num or 32
    args.kv_head_num = args.kv_head_num or args.head_num
    args.head_dim = args.head_dim or 128
  return args


def load_check(args, device):
  """Shape options, inputs and expected outputs of a --check file: (inputs on `device`, [expected or None, ...])."""
  if args.model_name not in CHECK_KEYS:
    raise SystemExit(f"--check knows the cases {sorted(CHECK_KEYS)}, not {args.model_name!r}")
  z = np.load(args.check, allow_pickle=False)
  B, S, H, D, seed = (int(z[k]) for k in ("B", "S", "H", "D", "seed"))
  args.batch_size, args.q_len, args.kv_len, args.head_num, args.head_dim = B, S, S, H, D
  g = torch.Generator(device="cpu")
  g.manual_seed(seed)
  dtype = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[args.type]
  inputs = [torch.randn(B, S, H, D, dtype=dtype, generator=g).to(device) for _ in range(3)]
  expected = []
  for key in CHECK_KEYS[args.model_name]:
    if key is not None and key not in z.files:
      raise SystemExit(f"{args.check} holds no array {key!r} (has {sorted(z.files)})")
    expected.append(None if key is None else torch.from_numpy(z[key]))
  return inputs, expected


def main(argv=None):
  args = parse_args(argv)
  if not torch.cuda.is_available():
    raise SystemExit("flashtensor_amd.run: no GPU visible")
  device = torch.device("cuda", torch.cuda.current_device())
  checked = load_check(args, device) if args.check else None
  print(" ".join(f"{k}={v!r}" for k, v in sorted(vars(args).items())))
  f, inputs, gflop, gb = build(args, device)
  if checked:
    inputs = checked[0]
    # SimA's results sit in fp16's subnormal range: its expected output is stored, and compared, in fp32
    res = ops.sima(*inputs, out_dtype=torch.float32) if args.model_name == "sima" else f(*inputs)
    torch.cuda.synchronize()
    for i, (o, r) in enumerate(zip(res if isinstance(res, tuple) else (res,), checked[1])):
      if r is not None:
        print(f"loss(out[{i}], ref[{i}], remove_zero=True)={loss(o.cpu(), r.reshape(o.shape), remove_zero=True)}")
  res = f(*inputs)
  torch.cuda.synchronize()
  if args.show_result:
    for i, r in enumerate(res if isinstance(res, tuple) else (res,)):
      print(f"out[{i}]={r}")
  perf(label="hip", f=f, args=inputs, gflops=gflop, mem_gb=gb, warmup=args.warmup, run=args.run)
  return res


if __name__ == "__main__":
  main()
