"""Backend interface of the reference (python/asuka/backend/builder.py:7-14): a Builder is constructed
around a kernel and `build_callable()` returns the function the harness calls with torch tensors
(cases/attn.py:120-127).  HipBuilder is the MI355X backend: its "kernel" is a case name plus
hyper-parameters instead of an MLIR sub-graph, and the callable launches the fused HIP kernels."""
from abc import ABC, abstractmethod
from typing import Any, Callable

from . import _lib
from .kernels import CASES, get_model


class Builder(ABC):

  def __init__(self, kernel) -> None:
    self.kernel = kernel

  @abstractmethod
  def build_callable(self) -> Callable[..., Any]:
    pass


class HipBuilder(Builder):
  """`HipBuilder('h2o').build_callable()` -> f(q, k, v) -> (out, h2o_score), positional arguments and
  result order of the case's forward (cases/kernels/h2o.py:18,38)."""

  def __init__(self, kernel, check_before_run=True, **hyper) -> None:
    if not isinstance(kernel, str) or kernel not in CASES:
      raise KeyError(f"unknown case {kernel!r}; have {sorted(CASES)}")
    super().__init__(kernel)
    self.check_before_run = check_before_run
    self.hyper = hyper

  def build_callable(self) -> Callable[..., Any]:
    _lib.ffi()  # fail here, not at the first call, when the HIP library is missing
    model = get_model(self.kernel, **self.hyper)
    if not self.check_before_run:
      return model.forward
    head_num, head_dim = model.head_num, model.head_dim
    if hasattr(model, "check_args"):  # cases whose arguments are not q, k, v

      def g(*args):
        model.check_args(*args)
        return model.forward(*args)

      return g

    def f(*args):
      for i, arg in enumerate(args[:3]):
        if arg.dim() != 4 or arg.shape[2] != head_num or arg.shape[3] != head_dim:
          raise RuntimeError(f"arg {i} need shape (B, S, {head_num}, {head_dim}) but got {tuple(arg.shape)}")
      return model.forward(*args)

    return f
