"""The C ABI without a GPU: the library loads, exports exactly what include/ft_abi.h declares, and
rejects bad arguments before anything is launched.  No compute call is made here."""
import ctypes
import os
import re

import pytest
import torch

import flashtensor_amd as ft
from flashtensor_amd import _lib
from flashtensor_amd._lib import FtAttnArgs, FtNoise, FtStrides

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
  return _lib.load()


def _declared():
  text = open(os.path.join(ROOT, "include", "ft_abi.h")).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(ft_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
  declared = _declared()
  assert declared == sorted(_lib.EXPORTS)
  for name in declared:
    assert getattr(lib, name) is not None
  header = open(os.path.join(ROOT, "include", "ft_abi.h")).read()
  version = int(re.search(r"#define FT_ABI_VERSION (\d+)", header).group(1))
  assert lib.ft_abi_version() == version == _lib.ABI_VERSION


def _args(**over):
  st = FtStrides(8 * 2 * 128, 2 * 128, 128)
  base = dict(q=0x1000, k=0x2000, v=0x3000, o=0x4000, sq=st, sk=st, sv=st, so=st, B=1, H=2, Sq=8, Skv=8, D=128,
              dtype=_lib.FT_F16, flags=_lib.FT_CAUSAL)
  base.update(over)
  return FtAttnArgs(**base)


@pytest.mark.parametrize("over,code,needle", [
    (dict(q=None), _lib.FT_EINVAL, "null"),
    (dict(o=None), _lib.FT_EINVAL, "null"),
    (dict(D=96), _lib.FT_EUNSUPPORTED, "head_dim"),
    (dict(dtype=_lib.FT_F32), _lib.FT_EUNSUPPORTED, "dtype"),
    (dict(Sq=0), _lib.FT_EINVAL, "shape"),
    (dict(Sq=16, Skv=8), _lib.FT_EINVAL, "Skv >= Sq"),
    (dict(q=0x1004), _lib.FT_EINVAL, "aligned"),
    (dict(sq=FtStrides(2048, 250, 128)), _lib.FT_EINVAL, "strides"),
    (dict(H=6, Hkv=4), _lib.FT_EINVAL, "grouping"),
    (dict(H=2, Hkv=4), _lib.FT_EINVAL, "grouping"),
])
def test_attn_rejects_bad_arguments_before_launch(lib, over, code, needle):
  a = _args(**over)
  assert lib.ft_attn_fwd(ctypes.byref(a), None, None) == code
  assert needle in lib.ft_last_error().decode()
  with pytest.raises((ValueError, _lib.FtError)):
    _lib.check(code)


def test_colstats_and_keyformer_argument_checks(lib):
  a = _args()
  need = lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(a))
  assert need == 1 * 2 * 8 * 4 == lib.ft_workspace_bytes(_lib.FT_OP_KEYFORMER, ctypes.byref(a))
  assert lib.ft_workspace_bytes(_lib.FT_OP_ATTN, ctypes.byref(a)) == 0
  assert lib.ft_attn_colstats_fwd(ctypes.byref(a), None, None, 0x5000, need, None) == _lib.FT_EINVAL
  assert lib.ft_attn_colstats_fwd(ctypes.byref(a), 0x6000, None, 0x5000, need - 1, None) == _lib.FT_EWORKSPACE
  assert "workspace" in lib.ft_last_error().decode()
  assert lib.ft_attn_colstats_fwd(ctypes.byref(a), 0x6000, None, None, need, None) == _lib.FT_EWORKSPACE
  noise = FtNoise(None, 0, 0, 0, 1)
  assert lib.ft_keyformer_fwd(ctypes.byref(a), None, 1.0, 0x6000, 0x5000, need, None) == _lib.FT_EINVAL
  assert lib.ft_keyformer_fwd(ctypes.byref(a), ctypes.byref(noise), 0.0, 0x6000, 0x5000, need, None) == _lib.FT_EINVAL
  assert "tau" in lib.ft_last_error().decode()
  assert lib.ft_keyformer_fwd(ctypes.byref(a), ctypes.byref(noise), 1.0, None, 0x5000, need, None) == _lib.FT_EINVAL


def test_softcap_corm_and_avgpool_argument_checks(lib):
  a = _args()
  assert lib.ft_attn_softcap_fwd(ctypes.byref(a), 0.0, None, None) == _lib.FT_EINVAL
  assert "softcap" in lib.ft_last_error().decode()
  assert lib.ft_attn_softcap_fwd(ctypes.byref(a), float("inf"), None, None) == _lib.FT_EINVAL
  assert lib.ft_attn_softcap_fwd(ctypes.byref(_args(D=96)), 50.0, None, None) == _lib.FT_EUNSUPPORTED
  need = lib.ft_workspace_bytes(_lib.FT_OP_CORM, ctypes.byref(a))
  assert need == 1 * 2 * 8 * 4
  assert lib.ft_corm_fwd(ctypes.byref(a), None, 0, None, None, 0x5000, need, None) == _lib.FT_EINVAL
  assert "corm_score" in lib.ft_last_error().decode()
  assert lib.ft_corm_fwd(ctypes.byref(a), 0x7000, 4, 0x6000, None, 0x5000, need, None) == _lib.FT_EINVAL  # row stride < Skv
  assert "corm_mask" in lib.ft_last_error().decode()
  assert lib.ft_corm_fwd(ctypes.byref(a), None, 0, 0x6000, None, 0x5000, need - 1, None) == _lib.FT_EWORKSPACE
  assert lib.ft_avgpool1d(None, 1, 8, 5, 0x2000, None) == _lib.FT_EINVAL
  assert lib.ft_avgpool1d(0x1000, 1, 8, 4, 0x2000, None) == _lib.FT_EINVAL
  assert "odd" in lib.ft_last_error().decode()
  assert lib.ft_avgpool1d(0x1000, 1, 8, 5, 0x1000, None) == _lib.FT_EINVAL
  assert lib.ft_avgpool1d(0x1000, 0, 8, 5, 0x2000, None) == _lib.FT_EINVAL


def test_grouped_query_argument_checks(lib):
  a = _args(H=4, Hkv=2)
  assert lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(a)) == 1 * 4 * 8 * 4 * 2   # normalisers + per-head sums
  assert lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(_args(H=4, Hkv=4))) == 1 * 4 * 8 * 4
  assert lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(_args(H=4))) == 1 * 4 * 8 * 4           # Hkv = 0 means H
  need = lib.ft_workspace_bytes(_lib.FT_OP_COLSTATS, ctypes.byref(a))
  assert lib.ft_attn_colstats_fwd(ctypes.byref(a), 0x6000, 0x7000, 0x5000, need, None) == _lib.FT_EUNSUPPORTED
  assert "grouped" in lib.ft_last_error().decode()
  assert lib.ft_attn_colstats_fwd(ctypes.byref(a), 0x6000, None, 0x5000, need - 1, None) == _lib.FT_EWORKSPACE
  noise = FtNoise(None, 0, 0, 0, 1)
  assert lib.ft_keyformer_fwd(ctypes.byref(a), ctypes.byref(noise), 1.0, 0x6000, 0x5000, need, None) == _lib.FT_EUNSUPPORTED
  assert lib.ft_corm_fwd(ctypes.byref(a), None, 0, 0x6000, None, 0x5000, need, None) == _lib.FT_EUNSUPPORTED


def test_linattn_and_topk_argument_checks(lib):
  st = FtStrides(64 * 2 * 64, 2 * 64, 64)
  a = _args(D=64, Sq=64, Skv=64, sq=st, sk=st, sv=st, so=st, flags=0)
  need = lib.ft_workspace_bytes(_lib.FT_OP_EA, ctypes.byref(a))
  assert need > 0 and need % 256 == 0
  assert lib.ft_linattn_fwd(ctypes.byref(a), 7, 1, _lib.FT_F16, 0x5000, need, None) == _lib.FT_EINVAL
  assert lib.ft_linattn_fwd(ctypes.byref(a), _lib.FT_OP_EA, 1, _lib.FT_F16, 0x5000, need - 1, None) == _lib.FT_EWORKSPACE
  b = _args(D=128, flags=0)
  assert lib.ft_linattn_fwd(ctypes.byref(b), _lib.FT_OP_SIMA, 1, _lib.FT_F16, 0x5000, 1 << 20, None) == _lib.FT_EUNSUPPORTED
  st32 = FtStrides(64 * 4 * 32, 4 * 32, 32)
  d32 = _args(D=32, H=4, Sq=64, Skv=64, sq=st32, sk=st32, sv=st32, so=st32, flags=0)
  need32 = lib.ft_workspace_bytes(_lib.FT_OP_SIMA, ctypes.byref(d32))
  assert need32 > 0 and lib.ft_linattn_fwd(ctypes.byref(d32), _lib.FT_OP_SIMA, 1, _lib.FT_F16, 0x5000, need32 - 1, None) == _lib.FT_EWORKSPACE
  odd = _args(D=32, H=3, Sq=64, Skv=64, sq=st32, sk=st32, sv=st32, so=st32, flags=0)
  assert lib.ft_linattn_fwd(ctypes.byref(odd), _lib.FT_OP_EA, 1, _lib.FT_F16, 0x5000, 1 << 20, None) == _lib.FT_EUNSUPPORTED
  far = _args(D=32, H=4, Sq=64, Skv=64, sq=st, sk=st, sv=st, so=st, flags=0)   # heads 64 apart: not adjacent pairs
  assert lib.ft_linattn_fwd(ctypes.byref(far), _lib.FT_OP_EA, 1, _lib.FT_F16, 0x5000, 1 << 20, None) == _lib.FT_EUNSUPPORTED
  c = _args(D=64, Sq=64, Skv=32, sq=st, sk=st, sv=st, so=st, flags=0)
  assert lib.ft_linattn_fwd(ctypes.byref(c), _lib.FT_OP_SIMA, 1, _lib.FT_F16, 0x5000, 1 << 20, None) == _lib.FT_EINVAL
  # types: bf16 and fp32 tensors are taken; the output is of the input type or fp32; fp32 strides in multiples of 4
  bf = _args(D=64, Sq=64, Skv=64, sq=st, sk=st, sv=st, so=st, flags=0, dtype=_lib.FT_BF16)
  assert lib.ft_linattn_fwd(ctypes.byref(bf), _lib.FT_OP_EA, 1, _lib.FT_BF16, 0x5000, need - 1, None) == _lib.FT_EWORKSPACE
  assert lib.ft_linattn_fwd(ctypes.byref(bf), _lib.FT_OP_EA, 1, _lib.FT_F16, 0x5000, need, None) == _lib.FT_EUNSUPPORTED
  assert "out_dtype" in lib.ft_last_error().decode()
  st4 = FtStrides(64 * 2 * 64 + 4, 2 * 64 + 4, 64)
  f32 = _args(D=64, Sq=64, Skv=64, sq=st4, sk=st4, sv=st4, so=st4, flags=0, dtype=_lib.FT_F32)
  assert lib.ft_linattn_fwd(ctypes.byref(f32), _lib.FT_OP_SIMA, 1, _lib.FT_F32, 0x5000, need - 1, None) == _lib.FT_EWORKSPACE
  assert lib.ft_linattn_fwd(ctypes.byref(f32), _lib.FT_OP_SIMA, 1, _lib.FT_F16, 0x5000, need, None) == _lib.FT_EUNSUPPORTED
  h4 = _args(D=64, Sq=64, Skv=64, sq=st4, sk=st4, sv=st4, so=st4, flags=0)   # 16-bit tensors need multiples of 8
  assert lib.ft_linattn_fwd(ctypes.byref(h4), _lib.FT_OP_EA, 1, _lib.FT_F16, 0x5000, need, None) == _lib.FT_EINVAL
  assert lib.ft_topk(None, 1, 8, 2, 0x1000, None) == _lib.FT_EINVAL
  assert lib.ft_topk(0x1000, 1, 8, 9, 0x2000, None) == _lib.FT_EINVAL
  assert lib.ft_topk(0x1000, 1, 32768, 16385, 0x2000, None) == _lib.FT_EUNSUPPORTED   # long rows: k <= 16384


def test_linear_block_argument_checks(lib):
  b = _lib.FtLinBlockArgs(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 2, 100, 4, 64, _lib.FT_F16)
  need = lib.ft_linattn_block_workspace_bytes(ctypes.byref(b), _lib.FT_OP_EA)
  C = 4 * 64
  assert need >= 2 * 100 * 4 * C * 2 + (32 << 20) and need % 256 == 0
  assert lib.ft_linattn_block_fwd(ctypes.byref(b), _lib.FT_OP_EA, 1, 0x10000, need - 1, None) == _lib.FT_EWORKSPACE
  assert lib.ft_linattn_block_fwd(ctypes.byref(b), 9, 1, 0x10000, need, None) == _lib.FT_EINVAL
  assert lib.ft_linattn_block_fwd(None, _lib.FT_OP_EA, 1, 0x10000, need, None) == _lib.FT_EINVAL
  bad = _lib.FtLinBlockArgs(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 2, 100, 4, 48, _lib.FT_F16)
  assert lib.ft_linattn_block_workspace_bytes(ctypes.byref(bad), _lib.FT_OP_EA) == 0
  assert "head_dim" in lib.ft_last_error().decode()
  # head_dim 32 runs as pairs of adjacent heads: an even number of them
  d32 = _lib.FtLinBlockArgs(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 2, 100, 4, 32, _lib.FT_F16)
  assert lib.ft_linattn_block_workspace_bytes(ctypes.byref(d32), _lib.FT_OP_EA) > 0
  odd32 = _lib.FtLinBlockArgs(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 2, 100, 3, 32, _lib.FT_F16)
  assert lib.ft_linattn_block_workspace_bytes(ctypes.byref(odd32), _lib.FT_OP_SIMA) == 0
  assert lib.ft_linattn_block_fwd(ctypes.byref(bad), _lib.FT_OP_SIMA, 1, 0x10000, need, None) == _lib.FT_EUNSUPPORTED
  odd = _lib.FtLinBlockArgs(0x1008, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 2, 100, 4, 64, _lib.FT_F16)
  assert lib.ft_linattn_block_fwd(ctypes.byref(odd), _lib.FT_OP_EA, 1, 0x10000, need, None) == _lib.FT_EINVAL
  f32 = _lib.FtLinBlockArgs(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 2, 100, 4, 64, _lib.FT_F32)
  assert lib.ft_linattn_block_workspace_bytes(ctypes.byref(f32), _lib.FT_OP_EA) >= 2 * 100 * 4 * C * 4 + (32 << 20)
  # narrow models in many short batches: the workspace also has to hold the two-launch form's partial matrices
  # (1120 floats per batch, chunk and head), more here than the library form's q / k / v
  many = _lib.FtLinBlockArgs(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 200000, 1, 4, 32, _lib.FT_F16)
  assert lib.ft_linattn_block_workspace_bytes(ctypes.byref(many), _lib.FT_OP_SIMA) >= 200000 * 4 * 1120 * 4
  nul = _lib.FtLinBlockArgs(0x1000, None, 0x3000, 0x4000, 0x5000, 0x6000, 2, 100, 4, 64, _lib.FT_F16)
  assert lib.ft_linattn_block_fwd(ctypes.byref(nul), _lib.FT_OP_EA, 1, 0x10000, need, None) == _lib.FT_EINVAL


def test_diag_probe_is_outside_the_product_abi_and_checks_its_arguments(lib):
  """The MFMA probe lives in libflashtensor_diag (include/ft_diag.h), not in the product library."""
  assert not hasattr(lib, "ft_probe_mfma") and not hasattr(lib, "ft_diag_probe_mfma")
  diag = _lib.load_diag()
  big = 65536
  assert diag.ft_diag_probe_mfma(None, big, 256, 10, 0x1000, None, None) == -1
  assert b"null" in diag.ft_diag_last_error()
  assert diag.ft_diag_probe_mfma(0x1008, big, 256, 10, 0x1000, None, None) == -1      # alignment
  assert diag.ft_diag_probe_mfma(0x1000, big - 1, 256, 10, 0x1000, None, None) == -1  # operand buffer too small
  assert b"FT_DIAG_PROBE_OPERAND_BYTES" in diag.ft_diag_last_error()
  assert diag.ft_diag_probe_mfma(0x1000, big, 0, 10, 0x1000, None, None) == -1
  assert diag.ft_diag_probe_mfma(0x1000, big, 256, 0, 0x1000, None, None) == -1
  assert diag.ft_diag_probe_mfma(0x1000, big, 256, 4000001, 0x1000, None, None) == -1  # iteration cap
  header = open(os.path.join(ROOT, "include", "ft_diag.h")).read()
  assert "#define FT_DIAG_PROBE_OPERAND_BYTES 65536" in header and "#define FT_DIAG_PROBE_MAX_ITERS 4000000" in header


def test_last_error_is_per_thread(lib):
  import threading
  seen, barrier = {}, threading.Barrier(4)

  def worker(i):
    barrier.wait()
    for _ in range(200):
      if i % 2:
        rc = lib.ft_topk(0x1000, 1, 8, 9 + i, 0x2000, None)           # k > S
        want = f"k={9 + i}"
      else:
        rc = lib.ft_avgpool1d(0x1000, 1, 8, 4 + i, 0x2000, None)      # even window
        want = "odd"
      msg = lib.ft_last_error().decode()
      if rc != _lib.FT_EINVAL or want not in msg:
        seen[i] = (rc, msg)
        return
    seen[i] = None

  threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
  for t in threads:
    t.start()
  for t in threads:
    t.join()
  assert seen == {0: None, 1: None, 2: None, 3: None}


def test_host_noise_twin_matches_oracle_stream(lib):
  import oracle
  E = ft.ops.seeded_exp_rand(2, 3, 17, 33, 987654321987, "cpu")
  ref = oracle.seeded_exp_rand(987654321987, 2, 3, 17, 33)
  assert torch.allclose(E, ref, rtol=1e-6, atol=0)


def test_operator_layer_validates_like_the_reference_backend():
  q = torch.zeros(1, 8, 2, 128, dtype=torch.float16)
  with pytest.raises(RuntimeError, match="need a GPU tensor"):
    ft.ops.attn(q, q, q)
  with pytest.raises(RuntimeError, match="need shape"):
    ft.ops.attn(q[0], q[0], q[0])
  with pytest.raises(KeyError):
    ft.HipBuilder("nope")
  f = ft.HipBuilder("h2o").build_callable()
  with pytest.raises(RuntimeError, match="arg 0 need shape"):
    f(torch.zeros(1, 8, 2, 64, dtype=torch.float16), q, q)
  assert sorted(ft.CASES) == ["attn", "corm", "ea", "ea_block", "gemma2", "h2o", "kf", "roco", "sima", "sima_block", "snapkv"]
  g = ft.HipBuilder("ea_block", head_num=2).build_callable()
  with pytest.raises(RuntimeError, match="arg 0 need shape"):
    g(torch.zeros(1, 8, 64, dtype=torch.float16), None, None, None, None)
  assert ft.get_model("snapkv").kernel_size == 5 and ft.get_model("gemma2").logit_softcapping == 50.0
  assert ft.get_model("kf").tau == 1.5 and ft.get_model("h2o").prepare.__doc__


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
  monkeypatch.setattr(_lib, "_lib", None)
  monkeypatch.setattr(_lib, "_ffi", None)
  monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libflashtensor_hip.so"))
  with pytest.raises(ImportError, match="not found"):
    _lib.load()
  with pytest.raises(ImportError, match="not found"):
    _lib.ffi()
  with pytest.raises(ImportError):
    ft.HipBuilder("attn").build_callable()


# ------------------------------------------------------------------ the pybind11 module over the same ABI

@pytest.fixture(scope="module")
def ffi():
  return _lib.ffi().kernels


def test_ffi_module_binds_every_declared_entry_point(ffi):
  """csrc/ffi_kernels.cpp exposes each function of include/ft_abi.h under its name without the ft_ prefix."""
  for name in _declared():
    assert callable(getattr(ffi, name[len("ft_"):])), name
  assert ffi.abi_version() == ffi.ABI_VERSION == _lib.ABI_VERSION
  assert (ffi.OK, ffi.EINVAL, ffi.EUNSUPPORTED, ffi.ELAUNCH, ffi.EWORKSPACE) == (0, -1, -2, -3, -4)
  assert (ffi.F16, ffi.BF16, ffi.F32, ffi.CAUSAL, ffi.FAST_LOGITS) == (0, 1, 2, 1, 2)
  assert (ffi.OP_ATTN, ffi.OP_COLSTATS, ffi.OP_KEYFORMER, ffi.OP_EA, ffi.OP_SIMA, ffi.OP_CORM) == (0, 1, 2, 3, 4, 5)


def _ffi_args(ffi, **over):
  st = (8 * 2 * 128, 2 * 128, 128)
  base = dict(q=0x1000, k=0x2000, v=0x3000, o=0x4000, sq=st, sk=st, sv=st, so=st, B=1, H=2, Sq=8, Skv=8, D=128,
              dtype=ffi.F16, flags=ffi.CAUSAL, Hkv=0)
  base.update(over)
  return ffi.AttnArgs(**base)


@pytest.mark.parametrize("over,exc,needle", [
    (dict(q=0), ValueError, "null"),
    (dict(o=0), ValueError, "null"),
    (dict(D=96), RuntimeError, "head_dim"),
    (dict(dtype=2), RuntimeError, "dtype"),
    (dict(Sq=0), ValueError, "shape"),
    (dict(Sq=16, Skv=8), ValueError, "Skv >= Sq"),
    (dict(q=0x1004), ValueError, "aligned"),
    (dict(sq=(2048, 250, 128)), ValueError, "strides"),
    (dict(H=6, Hkv=4), ValueError, "grouping"),
])
def test_ffi_module_maps_status_codes_to_exceptions(ffi, over, exc, needle):
  """FT_EINVAL -> ValueError (std::invalid_argument), anything else -> RuntimeError (std::runtime_error), the
  mapping of the reference's pybind layer (ffi/passes.cpp:81-83); nothing is launched for a rejected call."""
  with pytest.raises(exc, match=needle) as info:
    ffi.attn_fwd(_ffi_args(ffi, **over))
  if exc is RuntimeError:
    assert not isinstance(info.value, ValueError)
  assert "status" in str(info.value)


def test_ffi_module_workspace_and_validation_of_the_other_entry_points(ffi):
  a = _ffi_args(ffi, B=2, H=4, Sq=100, Skv=100)
  assert ffi.workspace_bytes(ffi.OP_ATTN, a) == 0
  assert ffi.workspace_bytes(ffi.OP_COLSTATS, a) == 2 * 4 * 100 * 4
  with pytest.raises(RuntimeError, match="workspace of 3200 bytes"):
    ffi.attn_colstats_fwd(a, 0x5000, 0, 0x6000, 16)
  with pytest.raises(ValueError, match="colsum"):
    ffi.attn_colstats_fwd(a, 0, 0, 0x6000, 3200)
  with pytest.raises(ValueError, match="tau"):
    ffi.keyformer_fwd(a, ffi.Noise(seed=1), 0.0, 0x5000, 0x6000, 3200)
  with pytest.raises(ValueError, match="softcap"):
    ffi.attn_softcap_fwd(a, -1.0)
  with pytest.raises(ValueError, match="odd"):
    ffi.avgpool1d(0x1000, 4, 64, 4, 0x2000)
  with pytest.raises(ValueError, match="top-k"):
    ffi.topk(0x1000, 4, 64, 65, 0x2000)
  with pytest.raises(RuntimeError, match="16384"):
    ffi.topk(0x1000, 4, 20000, 16385, 0x2000)
  with pytest.raises(ValueError, match="kind"):
    ffi.linattn_fwd(a, ffi.OP_ATTN, 1, ffi.F16, 0x6000, 1 << 20)
  with pytest.raises(ValueError, match="3 entries"):
    _ffi_args(ffi, sq=(1, 2))
  # the host twin of the noise stream runs without a GPU and matches the oracle's integer arithmetic
  import numpy as np
  import oracle
  buf = torch.empty(1, 2, 3, 5, dtype=torch.float32)
  ffi.noise_exp_fill_host(buf.data_ptr(), 1, 2, 3, 5, 99)
  np.testing.assert_allclose(buf.numpy(), oracle.seeded_exp_rand(99, 1, 2, 3, 5).numpy(), rtol=2e-6)
