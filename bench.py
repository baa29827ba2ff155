"""Benchmark of the fused attention + per-key score path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-configs] [--no-split] [--calibrate-copy]

A step is one H2O call (attention forward + column-statistics pass, the two launches behind
ft_attn_colstats_fwd) on B=1, H=32, S=4096, D=128 fp16 inputs already resident in HBM.  Prints ONE JSON
line: whole-step throughput in algorithmic TFLOP/s (two causal S x S x D contractions, 2 B H S^2 D FLOP,
whatever is recomputed internally), the roofline of the dominant kernel (the attention forward, timed
with events on the launch stream), the CPU baseline (the oracle's eager restatement on the host cores,
on a bounded subset of heads), and a per-configuration table for the five measured configurations.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

PEAK_MFMA_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# HBM-side bytes per launch of the attention kernel at the benchmark shape come from two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE, scaled by the readings of a 256 MiB tensor copy in the same run: --calibrate-copy).  They
# cannot be measured from inside this process, so the line quotes the last measurement, kept with the commit it
# was taken at in profiles/traffic.json, and says which commit that was.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(kernel):
  """(HBM bytes per launch, the commit the counters were read at) for `kernel`, or (None, None)."""
  try:
    with open(TRAFFIC_FILE) as f:
      entry = json.load(f)[kernel]
    return float(entry["fetch_bytes"]) + float(entry["write_bytes"]), entry["measured_at_commit"]
  except (OSError, KeyError, ValueError):
    return None, None


KERNEL_TIMING_ITERS = 300    # timed launches of the kernel-alone and step event loops, whatever --steps says
KERNEL_TIMING_WARMUP = 100
RAMP_SECONDS = 1.5           # untimed steps before the warm-up the caller asked for: clocks at their sustained level


def event_time_us(fn, iters=KERNEL_TIMING_ITERS, warmup=KERNEL_TIMING_WARMUP):
  """Average device time per call from events on torch's current stream (the stream the operators launch on)."""
  import torch
  for _ in range(warmup):
    fn()
  start = torch.cuda.Event(enable_timing=True)
  end = torch.cuda.Event(enable_timing=True)
  torch.cuda.synchronize()
  start.record()
  for _ in range(iters):
    fn()
  end.record()
  end.synchronize()
  return start.elapsed_time(end) * 1e3 / iters


def ramp(fn, seconds=RAMP_SECONDS):
  """Run fn back to back for about `seconds` of wall time (untimed); returns the time actually spent."""
  import torch
  t0 = time.perf_counter()
  while time.perf_counter() - t0 < seconds:
    for _ in range(50):
      fn()
    torch.cuda.synchronize()
  return time.perf_counter() - t0


def host_us_per_call(dev, calls=2000):
  """Host-side cost of one operator call (argument checks, two allocations, the ctypes call, the launch):
  wall time of un-synchronised calls on a problem small enough that the device never falls behind."""
  import torch
  from flashtensor_amd import ops
  q, k, v = (torch.randn(1, 64, 1, 128, dtype=torch.float16, device=dev) for _ in range(3))
  for _ in range(200):
    ops.attn(q, k, v)
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(calls):
    ops.attn(q, k, v)
  dt = time.perf_counter() - t0
  torch.cuda.synchronize()
  return dt / calls * 1e6


def per_config_table(dev, only=None, iters=100, splits=True):
  """µs per call, algorithmic TFLOP/s and GB/s with their roofline fractions for the five configurations
  (`only`: just the rows whose name contains that text)."""
  import torch
  from flashtensor_amd import ops
  rows = []

  def qkv(B, S, H, D):
    return tuple(torch.randn(B, S, H, D, dtype=torch.float16, device=dev) for _ in range(3))

  def add(name, shape, fn, flops, nbytes, split=False):
    if only is not None and only not in name:
      return
    try:
      us = event_time_us(fn, iters, warmup=max(20, iters // 4))
    except Exception as e:  # a row that cannot run (hipBLASLt absent, say) is reported, the line is still printed
      rows.append({"config": name, "shape": shape, "error": f"{type(e).__name__}: {e}"})
      return
    tf, gb = flops / us / 1e6, nbytes / us / 1e3
    rows.append({"config": name, "shape": shape, "us": round(us, 1), "tflops": round(tf, 1),
                 "mfma_frac": round(tf / PEAK_MFMA_TFLOPS, 4), "gbs": round(gb, 1), "hbm_frac": round(gb / PEAK_HBM_GBS, 4)})
    if split and splits:
      # The profiler's own durations run ~20 % long (tracing on), so only their proportions are used: the call's
      # event-timed microseconds divided among its kernels in those proportions.
      prof = kernel_split(fn)
      total = sum(v for v in prof.values() if isinstance(v, float))
      rows[-1]["kernels_us"] = ({k: round(us * v / total, 1) for k, v in prof.items()} if total > 0 and "error" not in prof else prof)

  def softmax_case(name, B, S, H, D, fn_of, extra_bytes=0, split=False):
    q, k, v = qkv(B, S, H, D)
    add(name, f"B{B} H{H} S{S} D{D}", fn_of(q, k, v), 2.0 * B * H * S * S * D, 4.0 * B * S * H * D * 2 + extra_bytes, split)

  softmax_case("1 attn", 1, 1024, 32, 128, lambda q, k, v: (lambda: ops.attn(q, k, v)))
  softmax_case("2 h2o+topk", 1, 2048, 32, 128,
               lambda q, k, v: (lambda: ops.topk(ops.h2o(q, k, v)[1], 256)), extra_bytes=32 * 2048 * 4)
  softmax_case("2' h2o", 1, 4096, 32, 128, lambda q, k, v: (lambda: ops.h2o(q, k, v)), extra_bytes=32 * 4096 * 4)
  # what reproducing the reference's fp16 rounding of the logits costs: the same call with the logits kept in fp32
  softmax_case("2' h2o, logits in fp32 (FT_FAST_LOGITS)", 1, 4096, 32, 128,
               lambda q, k, v: (lambda: ops.h2o(q, k, v, fast_logits=True)), extra_bytes=32 * 4096 * 4, split=True)
  softmax_case("3 keyformer seeded tau=1", 1, 4096, 32, 128,
               lambda q, k, v: (lambda: ops.keyformer(q, k, v, None, tau=1.0, seed=1)), extra_bytes=32 * 4096 * 4, split=True)
  if only is None or only in "3t keyformer tensor noise tau=1.5":
    er = 1 + torch.randn(1, 32, 4096, 4096, dtype=torch.float32, device=dev).abs()
    softmax_case("3t keyformer tensor noise tau=1.5", 1, 4096, 32, 128,
                 lambda q, k, v: (lambda: ops.keyformer(q, k, v, er, tau=1.5)),
                 # both passes read the visible (lower-triangular) half of the noise tensor, nothing above the diagonal
                 extra_bytes=2 * 32 * (4096 * 4097 // 2) * 4, split=True)
    del er
  softmax_case("4 roco", 4, 4096, 32, 128, lambda q, k, v: (lambda: ops.roco(q, k, v)), extra_bytes=2 * 4 * 32 * 4096 * 4)
  # the other cases of the reference's zoo at their prepare() defaults (B=1 H=32 S=4096 D=128)
  softmax_case("snapkv k=5", 1, 4096, 32, 128, lambda q, k, v: (lambda: ops.snapkv(q, k, v)), extra_bytes=32 * 4096 * 4)
  softmax_case("corm 1/(i+1)", 1, 4096, 32, 128, lambda q, k, v: (lambda: ops.corm(q, k, v)), extra_bytes=32 * 4096)
  softmax_case("gemma2 cap=50", 1, 4096, 32, 128, lambda q, k, v: (lambda: ops.gemma2(q, k, v)))
  q, k, v = qkv(1, 4096, 32, 128)
  kg, vg = k[:, :, :8].contiguous(), v[:, :, :8].contiguous()
  add("h2o grouped H32/Hkv8", "B1 H32 S4096 D128", lambda: ops.h2o(q, kg, vg), 2.0 * 32 * 4096 * 4096 * 128,
      (2 * q.numel() + 2 * kg.numel()) * 2.0 + 8 * 4096 * 4)
  q, k, v = qkv(8, 8192, 16, 64)
  lin_flops, lin_bytes = 2 * 2.0 * 8 * 16 * 8192 * 64 * 64, 4.0 * 8 * 16 * 8192 * 64 * 2
  add("5 ea", "B8 H16 S8192 D64", lambda: ops.ea(q, k, v), lin_flops, lin_bytes, split=True)
  add("5 sima", "B8 H16 S8192 D64", lambda: ops.sima(q, k, v), lin_flops, lin_bytes, split=True)
  del q, k, v
  # the whole function of bench/ea.mlir / bench/sima.mlir: hipBLASLt projections around the core (C = 1024)
  C, M = 16 * 64, 8 * 8192
  x = torch.randn(8, 8192, C, dtype=torch.float16, device=dev)
  wq = (torch.randn(3 * C, C, device=dev) / C ** 0.5).half()
  wo = (torch.randn(C, C, device=dev) / C ** 0.5).half()
  bq, bo = torch.zeros(3 * C, dtype=torch.float16, device=dev), torch.zeros(C, dtype=torch.float16, device=dev)
  blk_flops = lin_flops + 2.0 * M * (3 * C * C + C * C)
  blk_bytes = (2.0 * M * C + 4 * C * C + 4 * C) * 2  # x in, y out, the weights and biases once
  add("5b ea block (projections + core)", "B8 S8192 C1024 H16", lambda: ops.ea_block(x, wq, bq, wo, bo, 16), blk_flops, blk_bytes)
  add("5b sima block", "B8 S8192 C1024 H16", lambda: ops.sima_block(x, wq, bq, wo, bo, 16, normalize_q=False), blk_flops, blk_bytes)
  del x, wq, wo, bq, bo
  # the literal shape of bench/ea.mlir:2 (x [64,784,128], 4 heads of 32), in fp16: the two-launch form for narrow models
  C, M = 128, 64 * 784
  x = torch.randn(64, 784, C, dtype=torch.float16, device=dev)
  wq = (torch.randn(3 * C, C, device=dev) / C ** 0.5).half()
  wo = (torch.randn(C, C, device=dev) / C ** 0.5).half()
  bq, bo = torch.zeros(3 * C, dtype=torch.float16, device=dev), torch.zeros(C, dtype=torch.float16, device=dev)
  c_flops = 2 * 2.0 * 64 * 4 * 784 * 32 * 32 + 2.0 * M * 4 * C * C
  add("5c ea block, .mlir shape", "B64 S784 C128 H4 D32", lambda: ops.ea_block(x, wq, bq, wo, bo, 4),
      c_flops, (2.0 * M * C + 4 * C * C + 4 * C) * 2)
  add("5c sima block, .mlir shape", "B64 S784 C128 H4 D32", lambda: ops.sima_block(x, wq, bq, wo, bo, 4),
      c_flops, (2.0 * M * C + 4 * C * C + 4 * C) * 2)
  # ... and in the .mlir's own type
  xf, wqf, wof, bqf, bof = (t.float() for t in (x, wq, wo, bq, bo))
  add("5c ea block, .mlir shape and type (f32)", "B64 S784 C128 H4 D32", lambda: ops.ea_block(xf, wqf, bqf, wof, bof, 4),
      c_flops, (2.0 * M * C + 4 * C * C + 4 * C) * 4)
  add("5c sima block, .mlir shape and type (f32)", "B64 S784 C128 H4 D32", lambda: ops.sima_block(xf, wqf, bqf, wof, bof, 4),
      c_flops, (2.0 * M * C + 4 * C * C + 4 * C) * 4)
  return rows


def kernel_split(fn, iters=20):
  """Average device time per kernel name over `iters` calls of fn, from torch's profiler (kernel activity records):
  which launch of a multi-launch call the time goes to.  Diagnostic: returns an error entry where the profiler is
  not usable (another tracer attached, say)."""
  import torch
  try:
    from torch.profiler import ProfilerActivity, profile
    for _ in range(5):
      fn()
    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
      for _ in range(iters):
        fn()
      torch.cuda.synchronize()
    out = {}
    for ev in prof.key_averages():
      name, total = ev.key, getattr(ev, "device_time_total", None)
      if total is None:
        total = getattr(ev, "cuda_time_total", 0.0)
      if "ft::" not in name or not total:
        continue
      short = name.split("ft::", 1)[1].split("<", 1)[0].split("(", 1)[0]
      out[short] = round(out.get(short, 0.0) + total / iters, 1)
    return out or {"error": "no kernel records"}
  except Exception as e:
    return {"error": f"{type(e).__name__}: {e}"}


def mfma_probe(dev):
  """What the matrix pipe alone sustains on this chip: an MFMA-only loop (ft_diag_probe_mfma of the diagnostics
  library, include/ft_diag.h) on all-zero and on N(0,1) fp16 operands.  The chip is power-limited, so the second
  figure, not the published peak, is the rate the contractions of this workload could reach with nothing else running."""
  import ctypes
  import torch
  from flashtensor_amd import _lib
  diag = _lib.load_diag()
  cus = torch.cuda.get_device_properties(dev).multi_processor_count
  sink = torch.zeros(4, dtype=torch.float32, device=dev)
  clocks = torch.zeros(2, dtype=torch.int64, device=dev)
  stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
  out = {}
  for name, ops_ in (("zeros", torch.zeros(32768, dtype=torch.float16, device=dev)),
                     ("normal", torch.randn(32768, dtype=torch.float16, device=dev))):
    def run(iters):
      if diag.ft_diag_probe_mfma(ops_.data_ptr(), ops_.numel() * 2, cus, iters, sink.data_ptr(), clocks.data_ptr(), stream) != 0:
        raise RuntimeError(diag.ft_diag_last_error().decode())
    run(20000)  # ramp
    torch.cuda.synchronize()
    iters = 200000
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(); run(iters); e1.record(); e1.synchronize()
    ms = e0.elapsed_time(e1)
    c = clocks.cpu().tolist()
    out[name] = {"tflops": round(cus * 8 * iters * 4 * 32768 / ms / 1e9, 1), "shader_clock_mhz": round(100.0 * c[0] / max(1, c[1]))}
  return out


def cpu_baseline(B, S, H, D, heads):
  """The oracle's eager H2O forward on `heads` of the H heads (heads are independent), host cores."""
  import torch
  import oracle
  q, k, v = oracle.prepare_inputs(B, S, heads, D, seed=0)
  oracle.h2o_forward(q[:, :256], k[:, :256], v[:, :256])  # warm the thread pool
  t0 = time.perf_counter()
  oracle.h2o_forward(q, k, v)
  dt = time.perf_counter() - t0
  flops = 2.0 * B * heads * S * S * D
  return {"value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
          "sample": f"oracle.h2o_forward on {heads} of {H} heads at S={S} (heads are independent), {dt:.2f} s wall",
          "seconds": round(dt, 3), "host_cpus": os.cpu_count()}


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=500)
  ap.add_argument("--warmup", type=int, default=100)
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
  ap.add_argument("--no-configs", action="store_true", help="skip the per-configuration table")
  ap.add_argument("--cpu-heads", type=int, default=4)
  ap.add_argument("--only", default=None, help="per-configuration table: only the rows whose name contains this text")
  ap.add_argument("--config-iters", type=int, default=100, help="timed calls per row of the per-configuration table")
  ap.add_argument("--no-split", action="store_true",
                  help="per-configuration table without the per-kernel split (which attaches torch's profiler: leave it "
                       "out when the whole run is already under rocprofv3)")
  ap.add_argument("--calibrate-copy", action="store_true",
                  help="also run a 256 MiB device-to-device tensor copy a few times: under rocprofv3 --pmc its "
                       "FETCH_SIZE / WRITE_SIZE readings give the counter unit for the other kernels")
  args = ap.parse_args()
  if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
    sys.exit("bench.py: this path runs on ONE GPU (heads/batches shard with no communication); run with --gpus 1")

  import torch
  from flashtensor_amd import _lib, ops
  _lib.ffi()  # the HIP library (through its pybind11 module) is the only execution path
  if not torch.cuda.is_available():
    sys.exit("bench.py: no GPU visible")
  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)
  torch.manual_seed(0)

  B, H, S, D = 1, 32, 4096, 128
  # the CPU leg first, so that the GPU legs run back to back until the line is printed
  cpu = None if args.no_cpu else cpu_baseline(B, S, H, D, args.cpu_heads)
  q, k, v = (torch.randn(B, S, H, D, dtype=torch.float16, device=dev) for _ in range(3))
  flops = 2.0 * B * H * S * S * D
  alg_bytes = 4.0 * B * S * H * D * 2 + B * H * S * 4

  def step():
    return ops.h2o(q, k, v)

  if args.calibrate_copy:
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(5):
      dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

  ramp_s = ramp(step)  # untimed: a short run would otherwise be timed while the clocks are still settling
  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(args.steps):
    step()
  torch.cuda.synchronize()
  dt = (time.perf_counter() - t0) / args.steps

  # dominant kernel: the attention forward with its normaliser output, events on the launch stream; a fixed
  # number of launches, independent of --steps
  attn_us = event_time_us(lambda: ops.attn(q, k, v, return_lse=True))
  step_us = event_time_us(step)
  attn_tflops = flops / attn_us / 1e6
  host_us = host_us_per_call(dev)
  # the same step on inputs that rotate through 8 sets of q, k, v (805 MB, more than the 256 MB memory-side cache
  # holds), so that no launch finds its operands cached by the previous one
  sets = [tuple(torch.randn(B, S, H, D, dtype=torch.float16, device=dev) for _ in range(3)) for _ in range(8)]
  turn = [0]

  def cold_step():
    turn[0] = (turn[0] + 1) % len(sets)
    return ops.h2o(*sets[turn[0]])

  cold_us = event_time_us(cold_step)
  del sets

  traffic, traffic_commit = measured_traffic("attn_fwd_kernel")
  result = {
      "metric": "fused attn+score (H2O) algorithmic TFLOP/s at S=4096, 1 GPU",
      "value": round(flops / dt / 1e12, 2),
      "unit": "TFLOP/s",
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": round(dt * 1e3, 5),
      "ramp_s": round(ramp_s, 2),
      "host_us_per_call": round(host_us, 1),
      "us_per_step": round(dt * 1e6, 1),
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "f16",
      "data": "synthetic",
      "config": {"workload": "H2O fused attention + per-key column sums, causal, B=1 H=32 S=4096 D=128 fp16",
                 "launches_per_step": ["attn_fwd_kernel", "colstats_kernel"], "logits": "reference fp16 rounding"},
      "frac_of_fp16_mfma_peak": round(flops / dt / 1e12 / PEAK_MFMA_TFLOPS, 4),
      "algorithmic_gbs": round(alg_bytes / dt / 1e9, 1),
      "roofline": {"bound": "mfma", "kernel": "attn_fwd_kernel", "achieved": round(attn_tflops, 1), "peak": PEAK_MFMA_TFLOPS,
                   "unit": "TFLOP/s", "frac": round(attn_tflops / PEAK_MFMA_TFLOPS, 4), "traffic": traffic,
                   "traffic_measured_at": traffic_commit,
                   "us_per_launch": round(attn_us, 1), "algorithmic_flop_per_launch": flops,
                   "timed_launches": KERNEL_TIMING_ITERS},
      "kernels_us": {"attn_fwd_kernel": round(attn_us, 1), "colstats_kernel": round(step_us - attn_us, 1),
                     "step_events": round(step_us, 1), "step_events_cold_inputs": round(cold_us, 1)},
  }
  try:
    result["mfma_probe"] = mfma_probe(dev)
    result["mfma_probe"]["attn_fwd_kernel_frac_of_normal"] = round(attn_tflops / result["mfma_probe"]["normal"]["tflops"], 4)
  except Exception as e:  # diagnostic only: never costs the line
    result["mfma_probe"] = {"error": f"{type(e).__name__}: {e}"}
  if not args.no_configs:
    result["per_config"] = per_config_table(dev, args.only, args.config_iters, not args.no_split)
  result["cpu_baseline"] = cpu
  print(json.dumps(result))


if __name__ == "__main__":
  main()
