"""Prints the reference harness's loss lines (cases/attn_h2o.py:145-146, `loss(out, ref, remove_zero=True)`)
for one case of flashtensor_amd.run against the CPU oracle, then the timing line.  Not collected by pytest.

    python tests/run_case.py -m h2o --q_len 1024 --kv_len 1024
"""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

import oracle  # noqa: E402
from flashtensor_amd import run as cli  # noqa: E402
from flashtensor_amd.utils import loss, perf  # noqa: E402

ORACLE = {"attn": oracle.attn_forward, "h2o": oracle.h2o_forward, "roco": oracle.roco_forward, "snapkv": oracle.snapkv_forward,
          "gemma2": oracle.gemma2_forward, "ea": oracle.ea_forward, "sima": oracle.sima_forward,
          "kf": oracle.keyformer_forward, "corm": oracle.corm_forward}


def main():
  args = cli.parse_args(sys.argv[1:])
  print(" ".join(f"{k}={v!r}" for k, v in sorted(vars(args).items())))
  f, inputs, gflop, gb = cli.build(args, torch.device("cuda", torch.cuda.current_device()))
  res = f(*inputs)
  torch.cuda.synchronize()
  host = [t.cpu() for t in inputs]
  if args.model_name in cli.CASES_2D:
    fn = oracle.attn2d_forward if args.model_name == "attn_2d" else oracle.attn_h2o2d_forward
    ref = fn(*host, args.kv_head_num, args.head_num, args.head_dim, bool(args.masked))
  elif args.model_name.endswith("_block"):
    fn = oracle.ea_block_forward if args.model_name == "ea_block" else oracle.sima_block_forward
    ref = fn(*host, args.head_num or 16)
  else:
    ref = ORACLE[args.model_name](*host)
  res = res if isinstance(res, tuple) else (res,)
  ref = ref if isinstance(ref, tuple) else (ref,)
  for i, (o, r) in enumerate(zip(res, ref)):
    if o.dtype == torch.bool:
      print(f"out[{i}]: {(o.cpu() != r).sum().item()} of {o.numel()} decisions differ")
    else:
      print(f"loss(out[{i}], ref[{i}], remove_zero=True)={loss(o.cpu(), r, remove_zero=True)}")
  perf(label="hip", f=f, args=inputs, gflops=gflop, mem_gb=gb, warmup=args.warmup, run=args.run)


if __name__ == "__main__":
  main()
