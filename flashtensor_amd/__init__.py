"""flashtensor_amd: MI355X-native fused attention-variant kernels behind FlashTensor's operator boundary.

Only the hot path of the reference (monellz/FlashTensor) is here: the fused kernels of its attention
workloads, hand-written in HIP for gfx950 in `csrc/`, exported through the C ABI of `include/ft_abi.h`
(`libflashtensor_hip.so`), and a thin host mirror of the reference's backend interface
(`Builder.build_callable`, the case modules' `forward` / `prepare`).
"""
from . import kernels, ops  # noqa: F401
from .builder import Builder, HipBuilder  # noqa: F401
from .kernels import CASES, get_model  # noqa: F401
from .utils import loss, perf  # noqa: F401

__all__ = ["ops", "Builder", "HipBuilder", "CASES", "get_model", "loss", "perf"]
