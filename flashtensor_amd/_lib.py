"""Loaders of the native code: `ffi()` imports the pybind11 module ft_ffi (csrc/ffi_kernels.cpp) the operators
call through, `load()` binds libflashtensor_hip.so (the C ABI of include/ft_abi.h) directly with ctypes for
callers and tests that work at the level of the C ABI, `load_diag()` the diagnostics library.

The library is the product: if it is missing or fails to load these raise, there is no fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libflashtensor_hip.so")
DIAG_LIB_PATH = os.path.join(_HERE, "libflashtensor_diag.so")  # include/ft_diag.h: benchmark diagnostics, not product

FT_OK, FT_EINVAL, FT_EUNSUPPORTED, FT_ELAUNCH, FT_EWORKSPACE = 0, -1, -2, -3, -4
FT_F16, FT_BF16, FT_F32 = 0, 1, 2
FT_CAUSAL, FT_FAST_LOGITS = 1, 2
FT_OP_ATTN, FT_OP_COLSTATS, FT_OP_KEYFORMER, FT_OP_EA, FT_OP_SIMA, FT_OP_CORM = 0, 1, 2, 3, 4, 5
ABI_VERSION = 5

# every symbol include/ft_abi.h declares
EXPORTS = ("ft_abi_version", "ft_last_error", "ft_workspace_bytes", "ft_attn_fwd", "ft_attn_colstats_fwd", "ft_attn_colstats_fwd_static",
           "ft_keyformer_fwd", "ft_attn_softcap_fwd", "ft_corm_fwd", "ft_avgpool1d", "ft_linattn_fwd", "ft_topk",
           "ft_noise_exp_fill", "ft_noise_exp_fill_host", "ft_linattn_block_workspace_bytes", "ft_linattn_block_fwd")


class FtStrides(ctypes.Structure):
  _fields_ = [("b", ctypes.c_int64), ("s", ctypes.c_int64), ("h", ctypes.c_int64)]


class FtAttnArgs(ctypes.Structure):
  _fields_ = [("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("o", ctypes.c_void_p),
              ("sq", FtStrides), ("sk", FtStrides), ("sv", FtStrides), ("so", FtStrides),
              ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("Sq", ctypes.c_int32), ("Skv", ctypes.c_int32),
              ("D", ctypes.c_int32), ("dtype", ctypes.c_int32), ("flags", ctypes.c_uint32), ("Hkv", ctypes.c_int32)]


class FtLinBlockArgs(ctypes.Structure):
  _fields_ = [("x", ctypes.c_void_p), ("w_qkv", ctypes.c_void_p), ("b_qkv", ctypes.c_void_p), ("w_out", ctypes.c_void_p),
              ("b_out", ctypes.c_void_p), ("y", ctypes.c_void_p),
              ("B", ctypes.c_int32), ("S", ctypes.c_int32), ("H", ctypes.c_int32), ("D", ctypes.c_int32),
              ("dtype", ctypes.c_int32)]


class FtNoise(ctypes.Structure):
  _fields_ = [("exp_rand", ctypes.c_void_p), ("stride_b", ctypes.c_int64), ("stride_h", ctypes.c_int64),
              ("stride_row", ctypes.c_int64), ("seed", ctypes.c_uint64)]


class FtError(RuntimeError):
  """A kernel-library call failed; `.code` holds the FT_E* status."""

  def __init__(self, code, message):
    super().__init__(f"libflashtensor_hip: {message} (status {code})")
    self.code = code


_lib = None


def load():
  """Load the shared library once and declare the prototypes.  Raises if it has not been built."""
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} not found: build it with `python -m flashtensor_amd.build` "
                      "(the HIP library is the only execution path)")
  lib = ctypes.CDLL(LIB_PATH)
  vp, f32p = ctypes.c_void_p, ctypes.c_void_p
  args_p, noise_p = ctypes.POINTER(FtAttnArgs), ctypes.POINTER(FtNoise)
  lib.ft_abi_version.restype = ctypes.c_int
  lib.ft_abi_version.argtypes = []
  lib.ft_last_error.restype = ctypes.c_char_p
  lib.ft_last_error.argtypes = []
  lib.ft_workspace_bytes.restype = ctypes.c_size_t
  lib.ft_workspace_bytes.argtypes = [ctypes.c_int, args_p]
  lib.ft_attn_fwd.restype = ctypes.c_int
  lib.ft_attn_fwd.argtypes = [args_p, f32p, vp]
  lib.ft_attn_colstats_fwd.restype = ctypes.c_int
  lib.ft_attn_colstats_fwd.argtypes = [args_p, f32p, f32p, vp, ctypes.c_size_t, vp]
  lib.ft_attn_colstats_fwd_static.restype = ctypes.c_int
  lib.ft_attn_colstats_fwd_static.argtypes = [args_p, f32p, f32p, vp]
  lib.ft_keyformer_fwd.restype = ctypes.c_int
  lib.ft_keyformer_fwd.argtypes = [args_p, noise_p, ctypes.c_float, f32p, vp, ctypes.c_size_t, vp]
  lib.ft_attn_softcap_fwd.restype = ctypes.c_int
  lib.ft_attn_softcap_fwd.argtypes = [args_p, ctypes.c_float, f32p, vp]
  lib.ft_corm_fwd.restype = ctypes.c_int
  lib.ft_corm_fwd.argtypes = [args_p, f32p, ctypes.c_int64, vp, f32p, vp, ctypes.c_size_t, vp]
  lib.ft_avgpool1d.restype = ctypes.c_int
  lib.ft_avgpool1d.argtypes = [f32p, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, f32p, vp]
  lib.ft_linattn_fwd.restype = ctypes.c_int
  lib.ft_linattn_fwd.argtypes = [args_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, ctypes.c_size_t, vp]
  lib.ft_topk.restype = ctypes.c_int
  lib.ft_topk.argtypes = [f32p, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, vp, vp]
  lib.ft_noise_exp_fill.restype = ctypes.c_int
  lib.ft_noise_exp_fill.argtypes = [f32p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64, vp]
  lib.ft_noise_exp_fill_host.restype = ctypes.c_int
  lib.ft_noise_exp_fill_host.argtypes = [f32p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
  block_p = ctypes.POINTER(FtLinBlockArgs)
  lib.ft_linattn_block_workspace_bytes.restype = ctypes.c_size_t
  lib.ft_linattn_block_workspace_bytes.argtypes = [block_p, ctypes.c_int]
  lib.ft_linattn_block_fwd.restype = ctypes.c_int
  lib.ft_linattn_block_fwd.argtypes = [block_p, ctypes.c_int, ctypes.c_int, vp, ctypes.c_size_t, vp]
  if lib.ft_abi_version() != ABI_VERSION:
    raise ImportError(f"ABI version mismatch: library {lib.ft_abi_version()}, binding {ABI_VERSION}")
  _lib = lib
  return lib


def check(code):
  """Turn a non-zero status into an exception: bad arguments -> ValueError (the pybind layer of the
  reference maps std::invalid_argument the same way), anything else -> FtError (RuntimeError)."""
  if code == FT_OK:
    return
  msg = load().ft_last_error().decode("utf-8", "replace")
  if code == FT_EINVAL:
    raise ValueError(f"libflashtensor_hip: {msg}")
  raise FtError(code, msg)


_diag = None


def load_diag():
  """The diagnostics library of include/ft_diag.h (hardware probes for the benchmark); separate from the product ABI."""
  global _diag
  if _diag is None:
    if not os.path.exists(DIAG_LIB_PATH):
      raise ImportError(f"{DIAG_LIB_PATH} not found: build it with `python -m flashtensor_amd.build`")
    lib = ctypes.CDLL(DIAG_LIB_PATH)
    lib.ft_diag_last_error.restype = ctypes.c_char_p
    lib.ft_diag_last_error.argtypes = []
    lib.ft_diag_probe_mfma.restype = ctypes.c_int
    lib.ft_diag_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p,
                                       ctypes.c_void_p, ctypes.c_void_p]
    _diag = lib
  return _diag


_ffi = None


def ffi():
  """The pybind11 module over the C ABI (sub-module `kernels`), as the reference's asuka_ffi exposes its native code."""
  global _ffi
  if _ffi is None:
    if not os.path.exists(LIB_PATH):
      raise ImportError(f"{LIB_PATH} not found: build it with `python -m flashtensor_amd.build` "
                        "(the HIP library is the only execution path)")
    try:
      from . import ft_ffi
    except ImportError as e:
      raise ImportError(f"the pybind11 module ft_ffi is not built: run `python -m flashtensor_amd.build` ({e})") from e
    if ft_ffi.kernels.abi_version() != ABI_VERSION or ft_ffi.kernels.ABI_VERSION != ABI_VERSION:
      raise ImportError(f"ABI version mismatch: library {ft_ffi.kernels.abi_version()}, ft_ffi {ft_ffi.kernels.ABI_VERSION}, "
                        f"binding {ABI_VERSION}")
    _ffi = ft_ffi
  return _ffi
