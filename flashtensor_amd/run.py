"""Command-line harness in the manner of the reference's case scripts (cases/run.py:37-46 `-m <case>`,
cases/attn_h2o.py:84-164 shape options and the perf printout):

    python -m flashtensor_amd.run -m h2o [--batch_size 1] [--q_len 4096] [--kv_len 4096] [--type f16]
    python -m flashtensor_amd.run -m attn_h2o_2d --head_num 32 --kv_head_num 8 [--masked 1]

builds the case's callable through HipBuilder (or the 2-D harness classes), runs it on seeded N(0,1)
inputs and prints the timing line of `perf` with algorithmic GFLOP/s and GB/s.  Comparing against a CPU
definition is the test suite's job (tests/run_case.py prints the reference's loss lines).
"""
import argparse

import torch

from . import kernels
from .builder import HipBuilder
from .utils import perf

CASES_2D = {"attn_2d": kernels.Attn2D, "attn_h2o_2d": kernels.AttnH2O2D}


def build(args, device):
  """Returns (callable, input tensors, algorithmic GFLOP, algorithmic GB) for the parsed options."""
  dtype = torch.float16 if args.type == "f16" else torch.bfloat16
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
  ap.add_argument("--type", default="f16", choices=["f16", "bf16"])
  ap.add_argument("--run", type=int, default=10)
  ap.add_argument("--warmup", type=int, default=10)
  ap.add_argument("--show_result", action="store_true")
  args = ap.parse_args(argv)
  if args.model_name in CASES_2D:
    args.head_num = args.head_num or 32
    args.kv_head_num = args.kv_head_num or args.head_num
    args.head_dim = args.head_dim or 128
  return args


def main(argv=None):
  args = parse_args(argv)
  print(" ".join(f"{k}={v!r}" for k, v in sorted(vars(args).items())))
  if not torch.cuda.is_available():
    raise SystemExit("flashtensor_amd.run: no GPU visible")
  device = torch.device("cuda", torch.cuda.current_device())
  f, inputs, gflop, gb = build(args, device)
  res = f(*inputs)
  torch.cuda.synchronize()
  if args.show_result:
    for i, r in enumerate(res if isinstance(res, tuple) else (res,)):
      print(f"out[{i}]={r}")
  perf(label="hip", f=f, args=inputs, gflops=gflop, mem_gb=gb, warmup=args.warmup, run=args.run)
  return res


if __name__ == "__main__":
  main()
