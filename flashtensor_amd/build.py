"""Builds libflashtensor_hip.so (gfx950 only) in-tree with hipcc.

    python -m flashtensor_amd.build [--force]

One translation unit per kernel family, compiled in parallel, linked into a single shared library with
the C ABI of include/ft_abi.h.  hipcc cross-compiles, so this runs on hosts without a GPU.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libflashtensor_hip.so")
DIAG_LIB_PATH = os.path.join(HERE, "libflashtensor_diag.so")  # include/ft_diag.h: probes for the benchmark, not product
SOURCES = ["abi.hip", "attn_fwd.hip", "attn_fwd_f16_d128.hip", "attn_fwd_f16_d64.hip", "attn_fwd_bf16_d128.hip", "attn_fwd_bf16_d64.hip",
           "colstats.hip", "linattn.hip", "aux.hip", "linblock.hip", "linblock_small.hip"]
DIAG_SOURCES = ["diag.hip"]
FFI_SOURCE = "ffi_kernels.cpp"  # pybind11 module ft_ffi over the C ABI (plain C++: no device code, no torch headers)
HEADERS = ["device_common.hpp", "kernel_params.h", "noise.h", "attn_fwd_kernel.hpp", os.path.join("..", "..", "include", "ft_abi.h"),
           os.path.join("..", "..", "include", "ft_diag.h")]
# packed fp32 VALU ops are disabled on purpose: some forms have produced wrong results on this hardware
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument",
         # registers, scratch and spills of every kernel, written next to its object (see _resources): a spilled
         # register in a loop that keeps direct-to-LDS loads in flight costs far more than its reload
         "-Rpass-analysis=kernel-resource-usage"]
# The attention kernels take row maxima of MFMA results with plain fmaxf chains: without NaN honouring they become
# v_max3_f32 with no quieting moves, and stay visible to the compiler's hazard handling (no kernel relies on NaNs)
EXTRA_FLAGS = {src: ["-fno-honor-nans"] for src in ("attn_fwd_f16_d128.hip", "attn_fwd_f16_d64.hip", "attn_fwd_bf16_d128.hip", "attn_fwd_bf16_d64.hip")}


def _hipcc():
  rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
  cand = os.path.join(rocm, "bin", "hipcc")
  return cand if os.path.exists(cand) else "hipcc"


def _stale(target, deps):
  if not os.path.exists(target):
    return True
  t = os.path.getmtime(target)
  return any(os.path.getmtime(d) > t for d in deps)


def _resources(stderr):
  """{mangled kernel name: {"vgprs", "agprs", "scratch_bytes", "vgpr_spill", "sgpr_spill", "occupancy", "lds_bytes"}}
  from the compiler's kernel-resource-usage remarks."""
  import re
  keys = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes", "VGPRs Spill": "vgpr_spill",
          "SGPRs Spill": "sgpr_spill", "Occupancy [waves/SIMD]": "occupancy", "LDS Size [bytes/block]": "lds_bytes"}
  out, cur = {}, None
  for m in re.finditer(r"remark:\s+([A-Za-z][^:\n]*):\s+(\S+) \[-Rpass-analysis=kernel-resource-usage\]", stderr):
    name, val = m.group(1).strip(), m.group(2)
    if name == "Function Name":
      cur = out.setdefault(val, {})
    elif cur is not None and name in keys:
      cur[keys[name]] = int(val)
  return out


def resources_path(src):
  return os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".resources.json")


def _compile(src, force):
  obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
  deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, h) for h in HEADERS]
  if not force and not _stale(obj, deps):
    return obj, ""
  cmd = [_hipcc()] + FLAGS + EXTRA_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
  import json
  with open(resources_path(src), "w") as f:
    json.dump(_resources(res.stderr), f, indent=1, sort_keys=True)
  return obj, res.stderr


def _link(lib_path, objs, force):
  if force or _stale(lib_path, objs):
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
      raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")


def ffi_path():
  import sysconfig
  return os.path.join(HERE, "ft_ffi" + sysconfig.get_config_var("EXT_SUFFIX"))


def _build_ffi(force):
  """g++ on csrc/ffi_kernels.cpp against pybind11 and the Python headers, linked to libflashtensor_hip.so
  (found next to the module through an $ORIGIN run path)."""
  import sysconfig
  import pybind11
  out = ffi_path()
  src = os.path.join(CSRC, FFI_SOURCE)
  deps = [src, os.path.join(HERE, "..", "include", "ft_abi.h"), LIB_PATH]
  if not force and not _stale(out, deps):
    return out
  cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
         "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"], src, "-o", out,
         "-L" + HERE, "-lflashtensor_hip", "-Wl,-rpath,$ORIGIN"]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError(f"building ft_ffi failed:\n{res.stdout}\n{res.stderr}")
  return out


def build(force=False, verbose=True):
  os.makedirs(OBJ_DIR, exist_ok=True)
  sources = SOURCES + DIAG_SOURCES
  with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
    results = list(ex.map(lambda s: _compile(s, force), sources))
  objs = [o for o, _ in results]
  _link(LIB_PATH, objs[:len(SOURCES)], force)
  _link(DIAG_LIB_PATH, objs[len(SOURCES):], force)
  ffi = _build_ffi(force)
  if verbose:
    print(f"built {LIB_PATH}, {DIAG_LIB_PATH} and {ffi}")
  return LIB_PATH


if __name__ == "__main__":
  build(force="--force" in sys.argv)
