"""Case modules with the interface of the reference's workload zoo (cases/kernels/*.py): a class per
workload with `forward(...)` returning the same tensors in the same order, `prepare(...)` returning the
`{'input': {...}, 'output': [...]}` recipe, and `get_model()`.  `forward` runs the fused HIP kernels.
"""
import torch

from . import ops


class _Case:
  output = []

  def __init__(self, kv_head_num=32, head_num=32, head_dim=128):
    self.kv_head_num = kv_head_num
    self.head_num = head_num
    self.head_dim = head_dim
    self.hidden_size = head_num * head_dim
    self.kv_hidden_size = kv_head_num * head_dim
    self.group_size = self.head_num // self.kv_head_num
    assert self.group_size == 1  # as cases/kernels/attn.py:16

  def __call__(self, *args):
    return self.forward(*args)

  def eval(self):
    return self

  def _qkv(self, batch_size, q_len, kv_len, dtype, device):
    q = torch.randn(batch_size, q_len, self.head_num, self.head_dim, dtype=dtype, device=device)
    k = torch.randn(batch_size, kv_len, self.head_num, self.head_dim, dtype=dtype, device=device)
    v = torch.randn(batch_size, kv_len, self.head_num, self.head_dim, dtype=dtype, device=device)
    return {"q": q, "k": k, "v": v}

  def prepare(self, batch_size=1, q_len=4096, kv_len=4096, dtype=torch.float16, device=None):
    """Input recipe of cases/kernels/attn.py:36-49 (defaults B=1, S=4096, fp16, current GPU)."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    return {"input": self._qkv(batch_size, q_len, kv_len, dtype, device), "output": list(self.output)}


class Attn(_Case):
  """cases/kernels/attn.py: out = softmax(QK^T/sqrt(D) + causal) V."""
  output = ["out"]

  def forward(self, q, k, v):
    return ops.attn(q, k, v)


class H2O(_Case):
  """cases/kernels/h2o.py: (out, h2o_score)."""
  output = ["out", "h2o_score"]

  def forward(self, q, k, v):
    return ops.h2o(q, k, v)

  def heavy_hitters(self, h2o_score, k=None):
    """Top-k key indices per head (k defaults to S/8)."""
    return ops.topk(h2o_score, k or h2o_score.shape[-1] // 8)


class RoCo(_Case):
  """cases/kernels/roco.py: (out, roco_score, roco_sq_score)."""
  output = ["out", "roco_score", "roco_sq_score"]

  def forward(self, q, k, v):
    return ops.roco(q, k, v)

  @staticmethod
  def mean_var(roco_score, roco_sq_score, q_len):
    mean = roco_score / q_len
    return mean, roco_sq_score / q_len - mean * mean


class KeyFormer(_Case):
  """cases/kernels/kf.py: (out, kf_score); tau defaults to 1.5 as kf.py:8.  Passing exp_rand=None to
  forward draws the noise in-kernel from `seed`."""
  output = ["out", "kf_score"]

  def __init__(self, tau=1.5, kv_head_num=32, head_num=32, head_dim=128, seed=0):
    super().__init__(kv_head_num, head_num, head_dim)
    self.tau = tau
    self.seed = seed

  def forward(self, q, k, v, exp_rand=None):
    return ops.keyformer(q, k, v, exp_rand, tau=self.tau, seed=self.seed)

  def prepare(self, batch_size=1, q_len=4096, kv_len=4096, dtype=torch.float16, device=None):
    ret = super().prepare(batch_size, q_len, kv_len, dtype, device)
    dev = ret["input"]["q"].device
    ret["input"]["exp_rand"] = 1 + torch.randn(batch_size, self.head_num, q_len, kv_len, dtype=torch.float32, device=dev).abs()
    return ret


class SnapKV(_Case):
  """cases/kernels/snapkv.py: (out, snapkv_score); kernel_size defaults to 5 as snapkv.py:8."""
  output = ["out", "snapkv_score"]

  def __init__(self, kernel_size=5, kv_head_num=32, head_num=32, head_dim=128):
    super().__init__(kv_head_num, head_num, head_dim)
    self.kernel_size = kernel_size

  def forward(self, q, k, v):
    return ops.snapkv(q, k, v, kernel_size=self.kernel_size)


class Corm(_Case):
  """cases/kernels/corm.py: (out, corm_score bool).  Passing corm_mask=None to forward applies the
  prepare() thresholds 1 / (i + 1) without materialising them."""
  output = ["out", "corm_score"]

  def forward(self, q, k, v, corm_mask=None):
    return ops.corm(q, k, v, corm_mask)

  def prepare(self, batch_size=1, q_len=4096, kv_len=4096, dtype=torch.float16, device=None):
    ret = super().prepare(batch_size, q_len, kv_len, dtype, device)
    dev = ret["input"]["q"].device
    rows = torch.arange(1, q_len + 1, dtype=torch.float32, device=dev).unsqueeze(1)
    ret["input"]["corm_mask"] = torch.ones(q_len, kv_len, dtype=torch.float32, device=dev) / rows  # corm.py:47-49
    return ret


class Gemma2(_Case):
  """cases/kernels/gemma2.py: out, logits soft-capped at logit_softcapping (default 50, gemma2.py:8)."""
  output = ["out"]

  def __init__(self, logit_softcapping=50.0, kv_head_num=32, head_num=32, head_dim=128):
    super().__init__(kv_head_num, head_num, head_dim)
    self.logit_softcapping = logit_softcapping

  def forward(self, q, k, v):
    return ops.gemma2(q, k, v, softcap=self.logit_softcapping)


class Attn2D:
  """cases/attn.py:12-69: the harness form on 2-D activations, q [q_len, head_num * head_dim], k, v
  [kv_len, kv_head_num * head_dim] -> out [q_len, head_num * head_dim]; grouped queries when
  kv_head_num < head_num, `masked` selects the causal variant."""

  def __init__(self, kv_head_num, head_num, head_dim, masked):
    self.kv_head_num = kv_head_num
    self.head_num = head_num
    self.head_dim = head_dim
    self.masked = masked
    self.group_size = self.head_num // self.kv_head_num

  def __call__(self, *args):
    return self.forward(*args)

  def eval(self):
    return self

  def _views(self, q, k, v):
    return (q.view(1, q.shape[0], self.head_num, self.head_dim), k.view(1, k.shape[0], self.kv_head_num, self.head_dim),
            v.view(1, v.shape[0], self.kv_head_num, self.head_dim))

  def forward(self, q, k, v):
    q4, k4, v4 = self._views(q, k, v)
    return ops.attn(q4, k4, v4, causal=self.masked).view(q.shape[0], self.head_num * self.head_dim)


class AttnH2O2D(Attn2D):
  """cases/attn_h2o.py:11-81: (out [q_len, hidden], h2o_score [kv_head_num, kv_len])."""

  def forward(self, q, k, v):
    q4, k4, v4 = self._views(q, k, v)
    out, score = ops.h2o(q4, k4, v4, causal=self.masked)
    return out.view(q.shape[0], self.head_num * self.head_dim), score.view(self.kv_head_num, k.shape[0])


class EA(_Case):
  """Attention core of bench/ea.mlir:13-17 on [B,S,H,D] tensors."""
  output = ["out"]

  def __init__(self, kv_head_num=16, head_num=16, head_dim=64):
    super().__init__(kv_head_num, head_num, head_dim)

  def forward(self, q, k, v):
    return ops.ea(q, k, v)

  def prepare(self, batch_size=8, q_len=8192, kv_len=None, dtype=torch.float16, device=None):
    return super().prepare(batch_size, q_len, q_len, dtype, device)


class SimA(EA):
  """Attention core of bench/sima.mlir:13-17 on [B,S,H,D] tensors."""

  def __init__(self, kv_head_num=16, head_num=16, head_dim=64, normalize_q=True):
    super().__init__(kv_head_num, head_num, head_dim)
    self.normalize_q = normalize_q

  def forward(self, q, k, v):
    return ops.sima(q, k, v, normalize_q=self.normalize_q)


class EABlock:
  """The function of bench/ea.mlir:2-23 with its five arguments in order: x, the q/k/v Linear's weight and
  bias, the output Linear's weight and bias."""
  output = ["out"]

  def __init__(self, head_num=16, head_dim=64):
    self.head_num = head_num
    self.head_dim = head_dim
    self.hidden_size = head_num * head_dim

  def __call__(self, *args):
    return self.forward(*args)

  def eval(self):
    return self

  def check_args(self, x, *rest):
    if x.dim() != 3 or x.shape[2] != self.hidden_size:
      raise RuntimeError(f"arg 0 need shape (B, S, {self.hidden_size}) but got {tuple(x.shape)}")

  def forward(self, x, w_qkv, b_qkv, w_out, b_out):
    return ops.ea_block(x, w_qkv, b_qkv, w_out, b_out, self.head_num)

  def prepare(self, batch_size=8, q_len=8192, kv_len=None, dtype=torch.float16, device=None):
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    C = self.hidden_size
    x = torch.randn(batch_size, q_len, C, dtype=dtype, device=device)
    w_qkv = (torch.randn(3 * C, C, dtype=torch.float32, device=device) / C ** 0.5).to(dtype)
    b_qkv = (0.1 * torch.randn(3 * C, dtype=torch.float32, device=device)).to(dtype)
    w_out = (torch.randn(C, C, dtype=torch.float32, device=device) / C ** 0.5).to(dtype)
    b_out = (0.1 * torch.randn(C, dtype=torch.float32, device=device)).to(dtype)
    return {"input": {"x": x, "w_qkv": w_qkv, "b_qkv": b_qkv, "w_out": w_out, "b_out": b_out}, "output": self.output}


class SimABlock(EABlock):
  """The function of bench/sima.mlir:2-23."""

  def __init__(self, head_num=16, head_dim=64, normalize_q=True):
    super().__init__(head_num, head_dim)
    self.normalize_q = normalize_q

  def forward(self, x, w_qkv, b_qkv, w_out, b_out):
    return ops.sima_block(x, w_qkv, b_qkv, w_out, b_out, self.head_num, normalize_q=self.normalize_q)


CASES = {"attn": Attn, "h2o": H2O, "kf": KeyFormer, "roco": RoCo, "snapkv": SnapKV, "corm": Corm, "gemma2": Gemma2,
         "ea": EA, "sima": SimA, "ea_block": EABlock, "sima_block": SimABlock}


def get_model(name="attn", **kw):
  """`importlib.import_module('.' + name, 'kernels').get_model()` of cases/run.py:15-16, as one call."""
  if name not in CASES:
    raise KeyError(f"unknown case {name!r}; have {sorted(CASES)}")
  return CASES[name](**kw)
