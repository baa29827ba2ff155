// Host side of the C ABI declared in include/ft_abi.h: argument validation, kernel selection, launch.
// No device memory is allocated here and nothing synchronises; errors are reported through return
// codes plus a thread-local message, the C counterpart of the exceptions the reference's pybind layer
// throws (ffi/passes.cpp:81-83, ffi/ir.cpp:138) and of the shape / dtype checks of its TensorRT closure
// (python/asuka/backend/tensorrt/builder.py:104-111).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <atomic>
#include <cstring>
#include <mutex>

#include "../../include/ft_abi.h"
#include "kernel_params.h"
#include "noise.h"

namespace ft {
hipError_t launch_attn_fwd(const AttnKernelParams& p, int D, bool bf16, bool causal, bool emu, int kf, hipStream_t s);
hipError_t launch_colstats(const ColstatsKernelParams& p, int D, bool bf16, bool causal, bool emu, int mode,
                           hipStream_t s);
hipError_t launch_linattn(const FtAttnArgs& a, int kind, int normalize_q, int out_dtype, void* ws, hipStream_t s);
size_t linattn_workspace_bytes(const FtAttnArgs& a, int kind);
hipError_t launch_topk(const float* score, int64_t rows, int S, int k, int64_t* idx, hipStream_t s);
hipError_t launch_noise_fill(float* dst, int B, int H, int Sq, int Skv, uint64_t seed, hipStream_t s);
hipError_t launch_avgpool1d(const float* src, int64_t rows, int S, int kernel, float* dst, hipStream_t s);
hipError_t launch_group_mean(const float* src, int64_t groups, int group, int S, float* dst, hipStream_t s);
}  // namespace ft

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace

namespace ft {
// ft_last_error() for the translation units that hold entry points of their own
int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
}  // namespace ft

namespace {

int hip_fail(hipError_t e, const char* what) {
  return fail(FT_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
}

// ---- 16-bit float helpers (host) ------------------------------------------------------------------
float half_bits_to_float(uint16_t h) {
  _Float16 x;
  memcpy(&x, &h, 2);
  return (float)x;
}
uint16_t float_to_half_bits(float f) {
  _Float16 x = (_Float16)f;
  uint16_t h;
  memcpy(&h, &x, 2);
  return h;
}
float bf16_bits_to_float(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
uint16_t float_to_bf16_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// The eager reference divides the 16-bit QK^T tensor by sqrt(D) in 16-bit arithmetic, i.e. computes
// round16(float(x) / float(sqrt(D))) (cases/kernels/attn.py:29).  The kernels use one multiply instead:
// this finds the fp32 constant m near 1/sqrt(D) for which round16(float(x) * m) gives the same bits for
// every finite 16-bit x (exhaustive over all 65536 patterns; such an m exists for D = 64 and 128).
float tuned_logit_multiplier(int D, bool bf16) {
  static std::mutex mu;
  static float cache[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
  const int di = D == 128 ? 1 : 0;
  std::lock_guard<std::mutex> lock(mu);
  if (cache[bf16][di] != 0.f) return cache[bf16][di];
  const float c = (float)std::sqrt((double)D);
  const float rc = 1.0f / c;
  float best = rc;
  long best_bad = -1;
  for (int step = 0; step <= 16 && best_bad != 0; ++step) {
    for (int sign = -1; sign <= 1 && best_bad != 0; sign += 2) {
      if (step == 0 && sign == 1) continue;
      float m = rc;
      for (int s = 0; s < step; ++s) m = std::nextafterf(m, sign > 0 ? 1.0f : 0.0f);
      long bad = 0;
      for (uint32_t bits = 0; bits < 65536; ++bits) {
        const float x = bf16 ? bf16_bits_to_float((uint16_t)bits) : half_bits_to_float((uint16_t)bits);
        if (!std::isfinite(x)) continue;
        const uint16_t want = bf16 ? float_to_bf16_bits(x / c) : float_to_half_bits(x / c);
        const uint16_t got = bf16 ? float_to_bf16_bits(x * m) : float_to_half_bits(x * m);
        if (want != got) ++bad;
      }
      if (best_bad < 0 || bad < best_bad) {
        best_bad = bad;
        best = m;
      }
    }
  }
  cache[bf16][di] = best;
  return best;
}

// Packed-fp16 form of the division by sqrt(128) used by the fp16 fast paths: with hi = 0.70751953125 and
// lo = -0.0004127025604248047 (both fp16), fma16(h, hi, mul16(h, lo)) == 8 * f16(h / sqrt(128)) for every finite
// fp16 h whose quotient is at least 2.5e-3 in magnitude, and is within 2e-6 * 8 of it below (checked here over
// all 65536 inputs on first use; a logit that small moves a probability by 2e-6 relative).  D = 64 needs no
// constants: h / 8 is exact.
struct PackedLogitConstants {
  uint32_t hi2, lo2;  // the constant in both halves of a 32-bit word
  bool good;          // the exhaustive check passed
};
const PackedLogitConstants& packed_logit_constants() {
  // a function-local static is initialised exactly once per process, by whichever thread gets here first
  static const PackedLogitConstants consts = [] {
    const _Float16 hi = (_Float16)0.70751953125f, lo = (_Float16)-0.0004127025604248047f;
    bool ok = true;
    const float c = (float)std::sqrt(128.0);
    for (uint32_t bits = 0; bits < 65536 && ok; ++bits) {
      const float x = half_bits_to_float((uint16_t)bits);
      if (!std::isfinite(x)) continue;
      const double want = (double)(float)(_Float16)(x / c);
      const double cterm = (double)(float)(_Float16)((double)x * (double)(float)lo);
      const double got = (double)(float)(_Float16)((double)x * (double)(float)hi + cterm) / 8.0;
      if (got != want && (std::fabs(want) >= 2.5e-3 || std::fabs(got - want) > 2e-6)) ok = false;
    }
    const uint16_t hb = float_to_half_bits((float)hi), lb = float_to_half_bits((float)lo);
    return PackedLogitConstants{(uint32_t)hb | ((uint32_t)hb << 16), (uint32_t)lb | ((uint32_t)lb << 16), ok};
  }();
  return consts;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
bool stride_ok(const FtStrides& s) { return s.b % 8 == 0 && s.s % 8 == 0 && s.h % 8 == 0 && s.s > 0; }

int validate_attn(const FtAttnArgs* a, bool need_v_o) {
  if (!a) return fail(FT_EINVAL, "args is null");
  if (!a->q || !a->k) return fail(FT_EINVAL, "q / k pointer is null");
  if (need_v_o && (!a->v || !a->o)) return fail(FT_EINVAL, "v / o pointer is null");
  if (a->B < 1 || a->H < 1 || a->Sq < 1 || a->Skv < 1)
    return fail(FT_EINVAL, "bad shape B=%d H=%d Sq=%d Skv=%d", a->B, a->H, a->Sq, a->Skv);
  if (a->Hkv < 0 || (a->Hkv > 0 && (a->Hkv > a->H || a->H % a->Hkv != 0)))
    return fail(FT_EINVAL, "bad head grouping H=%d Hkv=%d (H must be a multiple of Hkv)", a->H, a->Hkv);
  if (a->D != 64 && a->D != 128) return fail(FT_EUNSUPPORTED, "head_dim %d not supported (64 or 128)", a->D);
  if (!packed_logit_constants().good) return fail(FT_EUNSUPPORTED, "internal: packed logit constants failed their exhaustive check");
  if (a->dtype != FT_F16 && a->dtype != FT_BF16) return fail(FT_EUNSUPPORTED, "dtype %d not supported (f16 or bf16)", a->dtype);
  if ((a->flags & FT_CAUSAL) && a->Skv < a->Sq)
    return fail(FT_EINVAL, "causal mask needs Skv >= Sq (got Sq=%d Skv=%d): rows without a visible key are undefined", a->Sq, a->Skv);
  if (!aligned16(a->q) || !aligned16(a->k) || (need_v_o && (!aligned16(a->v) || !aligned16(a->o))))
    return fail(FT_EINVAL, "q, k, v, o must be 16-byte aligned");
  if (!stride_ok(a->sq) || !stride_ok(a->sk) || (need_v_o && (!stride_ok(a->sv) || !stride_ok(a->so))))
    return fail(FT_EINVAL, "strides must be positive multiples of 8 elements with a contiguous head_dim axis");
  // tiles are fetched with 32-bit byte offsets from the (b, h) base of each operand
  if ((int64_t)a->Sq * a->sq.s * 2 >= 0x7fffffffLL || (int64_t)a->Skv * a->sk.s * 2 >= 0x7fffffffLL ||
      (need_v_o && (int64_t)a->Skv * a->sv.s * 2 >= 0x7fffffffLL))
    return fail(FT_EUNSUPPORTED, "sequence stride too large: S * stride_s must stay below 2^30 elements");
  const int64_t wgs = (int64_t)a->B * a->H * (((int64_t)(a->Sq > a->Skv ? a->Sq : a->Skv) + 63) / 64);
  if (wgs > 0x7fffffffLL) return fail(FT_EUNSUPPORTED, "problem too large for one launch");
  return FT_OK;
}

ft::Strides3 cvt(const FtStrides& s) { return ft::Strides3{s.b, s.s, s.h}; }
int group_of(const FtAttnArgs* a) { return a->Hkv > 0 ? a->H / a->Hkv : 1; }
int reject_groups(const FtAttnArgs* a, const char* what) {
  if (group_of(a) != 1) return fail(FT_EUNSUPPORTED, "%s does not take grouped queries (H=%d Hkv=%d)", what, a->H, a->Hkv);
  return FT_OK;
}

ft::AttnKernelParams attn_params(const FtAttnArgs* a, bool emu) {
  ft::AttnKernelParams p;
  memset(&p, 0, sizeof(p));
  p.q = (const uint16_t*)a->q;
  p.k = (const uint16_t*)a->k;
  p.v = (const uint16_t*)a->v;
  p.o = (uint16_t*)a->o;
  p.sq = cvt(a->sq);
  p.sk = cvt(a->sk);
  p.sv = cvt(a->sv);
  p.so = cvt(a->so);
  p.B = a->B;
  p.H = a->H;
  p.Sq = a->Sq;
  p.Skv = a->Skv;
  p.off = a->Skv - a->Sq;
  p.logit_mul = emu ? tuned_logit_multiplier(a->D, a->dtype == FT_BF16)
                    : (float)(1.4426950408889634 / std::sqrt((double)a->D));
  p.inv_tau = 1.f;
  p.group = group_of(a);
  p.pk_hi2 = packed_logit_constants().hi2;
  p.pk_lo2 = packed_logit_constants().lo2;
  return p;
}

ft::ColstatsKernelParams col_params(const FtAttnArgs* a, bool emu, const float* lse, float* colsum, float* colsumsq) {
  ft::ColstatsKernelParams p;
  memset(&p, 0, sizeof(p));
  p.q = (const uint16_t*)a->q;
  p.k = (const uint16_t*)a->k;
  p.sq = cvt(a->sq);
  p.sk = cvt(a->sk);
  p.lse = lse;
  p.colsum = colsum;
  p.colsumsq = colsumsq;
  p.B = a->B;
  p.H = a->H;
  p.Sq = a->Sq;
  p.Skv = a->Skv;
  p.off = a->Skv - a->Sq;
  p.logit_mul = emu ? tuned_logit_multiplier(a->D, a->dtype == FT_BF16)
                    : (float)(1.4426950408889634 / std::sqrt((double)a->D));
  p.inv_tau = 1.f;
  p.group = group_of(a);
  p.pk_hi2 = packed_logit_constants().hi2;
  p.pk_lo2 = packed_logit_constants().lo2;
  return p;
}

size_t lse_bytes(const FtAttnArgs* a) { return (size_t)a->B * a->H * a->Sq * sizeof(float); }
// grouped queries: the per-query-head column sums live in the workspace before their group mean is taken
size_t colstats_bytes(const FtAttnArgs* a) {
  return lse_bytes(a) + (group_of(a) > 1 ? (size_t)a->B * a->H * a->Skv * sizeof(float) : 0);
}


int validate_colstats(const FtAttnArgs* a, const float* colsum, const float* colsumsq) {
  if (int rc = validate_attn(a, true)) return rc;
  if (!colsum) return fail(FT_EINVAL, "colsum pointer is null");
  const int group = group_of(a);
  if (group > 1 && colsumsq) return fail(FT_EUNSUPPORTED, "sum of squares is not defined per query head under grouped queries");
  if (group > 1 && (int64_t)a->B * a->Hkv > 65535) return fail(FT_EUNSUPPORTED, "too many k/v heads for the group mean");
  return FT_OK;
}

// attention pass (writes the row normalisers to the scratch), column pass, group mean when grouped; `ws` holds
// colstats_bytes(a) bytes.  Every scratch element that is read has been written earlier in the same call.
int run_colstats(const FtAttnArgs* a, float* colsum, float* colsumsq, void* ws, void* stream) {
  const int group = group_of(a);
  const bool emu = !(a->flags & FT_FAST_LOGITS);
  const bool causal = a->flags & FT_CAUSAL;
  float* lse = static_cast<float*>(ws);
  float* per_head = group > 1 ? lse + (size_t)a->B * a->H * a->Sq : colsum;
  ft::AttnKernelParams p = attn_params(a, emu);
  p.lse = lse;
  hipError_t e = ft::launch_attn_fwd(p, a->D, a->dtype == FT_BF16, causal, emu, ft::kKfNone, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "attn_fwd launch");
  ft::ColstatsKernelParams c = col_params(a, emu, lse, per_head, colsumsq);
  e = ft::launch_colstats(c, a->D, a->dtype == FT_BF16, causal, emu, colsumsq ? ft::kStatSumSq : ft::kStatSum,
                          (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "colstats launch");
  if (group > 1) {
    e = ft::launch_group_mean(per_head, (int64_t)a->B * a->Hkv, group, a->Skv, colsum, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "group mean launch");
  }
  return FT_OK;
}

// Scratch of ft_attn_colstats_fwd_static: device memory that is part of the loaded code object, so that the
// entry point never calls an allocator.  Each GPU holds its own copy at its own address; the name below is a
// host-side handle, not a device address: the address is looked up once per device (with that device current)
// and only that pointer is handed to kernels.
static __device__ __align__(256) unsigned char scratch[FT_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];  // zero-initialised; a racing first call stores the same address twice

int static_scratch(void** out, hipStream_t stream) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  // the buffer handed out is the current device's copy: a stream of another device would run the kernels there
  // with this device's address
  int sdev = dev;
  if (stream && hipStreamGetDevice(stream, &sdev) == hipSuccess && sdev != dev)
    return fail(FT_EINVAL, "stream belongs to device %d, the current device is %d", sdev, dev);
  if (dev < 0 || dev >= kMaxDevices) return fail(FT_EUNSUPPORTED, "device index %d beyond the %d this entry point tracks", dev, kMaxDevices);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return FT_OK;
}

}  // namespace

extern "C" {

int ft_abi_version(void) { return FT_ABI_VERSION; }

const char* ft_last_error(void) { return g_err; }

size_t ft_workspace_bytes(int op, const FtAttnArgs* a) {
  if (!a) return 0;
  switch (op) {
    case FT_OP_ATTN:
      return 0;
    case FT_OP_COLSTATS:
      return colstats_bytes(a);
    case FT_OP_KEYFORMER:
    case FT_OP_CORM:
      return lse_bytes(a);
    case FT_OP_EA:
    case FT_OP_SIMA:
      return ft::linattn_workspace_bytes(*a, op);
    default:
      return 0;
  }
}

int ft_attn_fwd(const FtAttnArgs* a, float* lse, void* stream) {
  if (int rc = validate_attn(a, true)) return rc;
  const bool emu = !(a->flags & FT_FAST_LOGITS);
  ft::AttnKernelParams p = attn_params(a, emu);
  p.lse = lse;
  hipError_t e = ft::launch_attn_fwd(p, a->D, a->dtype == FT_BF16, a->flags & FT_CAUSAL, emu, ft::kKfNone, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "attn_fwd launch");
  return FT_OK;
}

int ft_attn_colstats_fwd(const FtAttnArgs* a, float* colsum, float* colsumsq, void* workspace, size_t workspace_bytes,
                         void* stream) {
  if (int rc = validate_colstats(a, colsum, colsumsq)) return rc;
  const size_t need = colstats_bytes(a);
  if (!workspace || workspace_bytes < need)
    return fail(FT_EWORKSPACE, "workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (reinterpret_cast<uintptr_t>(workspace) & 3u) return fail(FT_EINVAL, "workspace must be 4-byte aligned");
  return run_colstats(a, colsum, colsumsq, workspace, stream);
}

int ft_attn_colstats_fwd_static(const FtAttnArgs* a, float* colsum, float* colsumsq, void* stream) {
  if (int rc = validate_colstats(a, colsum, colsumsq)) return rc;
  const size_t need = colstats_bytes(a);
  if (need > (size_t)FT_STATIC_SCRATCH_BYTES)
    return fail(FT_EWORKSPACE, "problem needs %zu bytes of scratch, the static buffer holds %zu: use ft_attn_colstats_fwd with a workspace",
                need, (size_t)FT_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws, (hipStream_t)stream)) return rc;
  return run_colstats(a, colsum, colsumsq, ws, stream);
}

int ft_keyformer_fwd(const FtAttnArgs* a, const FtNoise* noise, float tau, float* kf_score, void* workspace,
                     size_t workspace_bytes, void* stream) {
  if (int rc = validate_attn(a, true)) return rc;
  if (int rc = reject_groups(a, "keyformer")) return rc;
  if (!noise) return fail(FT_EINVAL, "noise descriptor is null");
  if (!kf_score) return fail(FT_EINVAL, "kf_score pointer is null");
  if (!(tau > 0.f) || !std::isfinite(tau)) return fail(FT_EINVAL, "tau must be positive and finite (got %g)", (double)tau);
  if (!workspace || workspace_bytes < lse_bytes(a))
    return fail(FT_EWORKSPACE, "workspace of %zu bytes needed, got %zu", lse_bytes(a), workspace ? workspace_bytes : (size_t)0);
  if (reinterpret_cast<uintptr_t>(workspace) & 3u) return fail(FT_EINVAL, "workspace must be 4-byte aligned");
  const bool tensor = noise->exp_rand != nullptr;
  if (tensor && (noise->stride_row < a->Skv || (reinterpret_cast<uintptr_t>(noise->exp_rand) & 3u)))
    return fail(FT_EINVAL, "exp_rand needs a contiguous last axis and row stride >= Skv");
  const bool emu = !(a->flags & FT_FAST_LOGITS);
  const bool causal = a->flags & FT_CAUSAL;
  float* lse_kf = static_cast<float*>(workspace);
  ft::AttnKernelParams p = attn_params(a, emu);
  p.lse = nullptr;
  p.lse_kf = lse_kf;
  p.inv_tau = 1.f / tau;
  p.seed = noise->seed;
  if (tensor) {
    p.exp_rand = noise->exp_rand;
    p.er_sb = noise->stride_b;
    p.er_sh = noise->stride_h;
    p.er_sr = noise->stride_row;
    p.er_vec4 = aligned16(noise->exp_rand) && noise->stride_b % 4 == 0 && noise->stride_h % 4 == 0 && noise->stride_row % 4 == 0;
  }
  // seeded noise, fp16, reference rounding: the packed path (tau == 1 needs 1 / E only; tau >= 0.25 keeps
  // the perturbed sum inside fp32 range under the plain softmax's stabiliser); otherwise the generic path
  int amode = tensor ? ft::kKfTensor : ft::kKfSeeded, cmode = tensor ? ft::kStatKfTensor : ft::kStatKfSeeded;
  // noise rows that can be fetched in 16-byte chunks through a buffer descriptor of the (b, h) slice: the attention
  // pass lands them in LDS a tile ahead
  if (tensor && p.er_vec4 && a->Skv % 4 == 0 && (int64_t)a->Sq * noise->stride_row * 4 < (int64_t)0x7fffffff)
    amode = ft::kKfTensorLds;
  if (!tensor && emu && a->dtype == FT_F16) {
    if (tau == 1.f) {
      amode = ft::kKfSeededTau1;
      cmode = ft::kStatKfSeededTau1;
    } else if (tau >= 0.25f) {
      amode = ft::kKfSeededFast;
      cmode = ft::kStatKfSeededFast;
    }
  }
  hipError_t e = ft::launch_attn_fwd(p, a->D, a->dtype == FT_BF16, causal, emu, amode, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "attn_fwd (keyformer) launch");
  ft::ColstatsKernelParams c = col_params(a, emu, lse_kf, kf_score, nullptr);
  c.inv_tau = 1.f / tau;
  c.seed = noise->seed;
  if (tensor) {
    c.exp_rand = noise->exp_rand;
    c.er_sb = noise->stride_b;
    c.er_sh = noise->stride_h;
    c.er_sr = noise->stride_row;
  }
  e = ft::launch_colstats(c, a->D, a->dtype == FT_BF16, causal, emu, cmode, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "colstats (keyformer) launch");
  return FT_OK;
}

int ft_attn_softcap_fwd(const FtAttnArgs* a, float softcap, float* lse, void* stream) {
  if (int rc = validate_attn(a, true)) return rc;
  if (!(softcap > 0.f) || !std::isfinite(softcap)) return fail(FT_EINVAL, "softcap must be positive and finite (got %g)", (double)softcap);
  const bool emu = !(a->flags & FT_FAST_LOGITS);
  ft::AttnKernelParams p = attn_params(a, emu);
  p.lse = lse;
  p.softcap = softcap;
  hipError_t e = ft::launch_attn_fwd(p, a->D, a->dtype == FT_BF16, a->flags & FT_CAUSAL, emu, ft::kKfSoftcap, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "attn_fwd (softcap) launch");
  return FT_OK;
}

int ft_corm_fwd(const FtAttnArgs* a, const float* corm_mask, int64_t mask_row_stride, uint8_t* corm_score, float* margin,
                void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = validate_attn(a, true)) return rc;
  if (int rc = reject_groups(a, "corm")) return rc;
  if (!corm_score) return fail(FT_EINVAL, "corm_score pointer is null");
  if (corm_mask && (mask_row_stride < a->Skv || (reinterpret_cast<uintptr_t>(corm_mask) & 3u)))
    return fail(FT_EINVAL, "corm_mask needs a contiguous last axis and row stride >= Skv");
  if (!workspace || workspace_bytes < lse_bytes(a))
    return fail(FT_EWORKSPACE, "workspace of %zu bytes needed, got %zu", lse_bytes(a), workspace ? workspace_bytes : (size_t)0);
  if (reinterpret_cast<uintptr_t>(workspace) & 3u) return fail(FT_EINVAL, "workspace must be 4-byte aligned");
  const bool emu = !(a->flags & FT_FAST_LOGITS);
  const bool causal = a->flags & FT_CAUSAL;
  float* lse = static_cast<float*>(workspace);
  ft::AttnKernelParams p = attn_params(a, emu);
  p.lse = lse;
  hipError_t e = ft::launch_attn_fwd(p, a->D, a->dtype == FT_BF16, causal, emu, ft::kKfNone, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "attn_fwd launch");
  ft::ColstatsKernelParams c = col_params(a, emu, lse, margin, nullptr);
  c.keep = corm_score;
  if (corm_mask) {
    c.exp_rand = corm_mask;
    c.er_sr = mask_row_stride;
  }
  e = ft::launch_colstats(c, a->D, a->dtype == FT_BF16, causal, emu, corm_mask ? ft::kStatCormTensor : ft::kStatCormRule,
                          (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "colstats (corm) launch");
  return FT_OK;
}

int ft_avgpool1d(const float* src, int64_t rows, int32_t S, int32_t kernel, float* dst, void* stream) {
  if (!src || !dst) return fail(FT_EINVAL, "src / dst pointer is null");
  if (src == dst) return fail(FT_EINVAL, "src and dst must not alias");
  if (rows < 1 || S < 1) return fail(FT_EINVAL, "bad shape rows=%lld S=%d", (long long)rows, S);
  if (kernel < 1 || (kernel & 1) == 0) return fail(FT_EINVAL, "kernel must be odd and positive (got %d): only then is the output as long as the input", kernel);
  if (rows > 65535) return fail(FT_EUNSUPPORTED, "too many rows");
  hipError_t e = ft::launch_avgpool1d(src, rows, S, kernel, dst, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "avgpool1d launch");
  return FT_OK;
}

int ft_linattn_fwd(const FtAttnArgs* a, int kind, int normalize_q, int out_dtype, void* workspace, size_t workspace_bytes,
                   void* stream) {
  if (!a) return fail(FT_EINVAL, "args is null");
  if (kind != FT_OP_EA && kind != FT_OP_SIMA) return fail(FT_EINVAL, "kind must be FT_OP_EA or FT_OP_SIMA");
  if (!a->q || !a->k || !a->v || !a->o) return fail(FT_EINVAL, "q / k / v / o pointer is null");
  if (a->B < 1 || a->H < 1 || a->Sq < 1 || a->Skv != a->Sq)
    return fail(FT_EINVAL, "bad shape B=%d H=%d Sq=%d Skv=%d (linear attention needs Sq == Skv)", a->B, a->H, a->Sq, a->Skv);
  if (a->Hkv != 0 && a->Hkv != a->H) return fail(FT_EUNSUPPORTED, "linear attention does not take grouped queries (H=%d Hkv=%d)", a->H, a->Hkv);
  if (a->D != 64 && a->D != 32)
    return fail(FT_EUNSUPPORTED, "head_dim %d not supported by the linear-attention kernels (64, or 32 in adjacent pairs)", a->D);
  if (a->D == 32 && ((a->H & 1) || a->sq.h != 32 || a->sk.h != 32 || a->sv.h != 32 || a->so.h != 32))
    return fail(FT_EUNSUPPORTED, "head_dim 32 needs an even number of heads stored 32 elements apart (H=%d)", a->H);
  if (a->dtype != FT_F16 && a->dtype != FT_BF16 && a->dtype != FT_F32)
    return fail(FT_EUNSUPPORTED, "dtype %d not supported by the linear-attention kernels (f16, bf16 or f32)", a->dtype);
  if (out_dtype != a->dtype && out_dtype != FT_F32)
    return fail(FT_EUNSUPPORTED, "out_dtype must be the input type or f32 (got %d for inputs of type %d)", out_dtype, a->dtype);
  if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->o))
    return fail(FT_EINVAL, "q, k, v, o must be 16-byte aligned");
  // rows are moved in 16-byte pieces: strides in multiples of 8 elements for 16-bit tensors, of 4 for fp32 ones
  const int64_t in_mul = a->dtype == FT_F32 ? 4 : 8, out_mul = out_dtype == FT_F32 ? 4 : 8;
  auto strides_ok = [](const FtStrides& s, int64_t m) { return s.b % m == 0 && s.s % m == 0 && s.h % m == 0 && s.s > 0; };
  if (!strides_ok(a->sq, in_mul) || !strides_ok(a->sk, in_mul) || !strides_ok(a->sv, in_mul) || !strides_ok(a->so, out_mul))
    return fail(FT_EINVAL, "strides must be positive multiples of 16 bytes with a contiguous head_dim axis");
  const int64_t esz = a->dtype == FT_F32 ? 4 : 2;
  if ((int64_t)a->Sq * a->sq.s * esz >= 0x7fffffffLL || (int64_t)a->Sq * a->sk.s * esz >= 0x7fffffffLL ||
      (int64_t)a->Sq * a->sv.s * esz >= 0x7fffffffLL)
    return fail(FT_EUNSUPPORTED, "sequence stride too large: S * stride_s must stay below 2^31 bytes");
  const size_t need = ft::linattn_workspace_bytes(*a, kind);
  if (!workspace || workspace_bytes < need)
    return fail(FT_EWORKSPACE, "workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(FT_EINVAL, "workspace must be 16-byte aligned");
  hipError_t e = ft::launch_linattn(*a, kind, normalize_q, out_dtype, workspace, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "linattn launch");
  return FT_OK;
}

int ft_topk(const float* score, int64_t rows, int32_t S, int32_t k, int64_t* idx, void* stream) {
  if (!score || !idx) return fail(FT_EINVAL, "score / idx pointer is null");
  if (rows < 1 || S < 1 || k < 1 || k > S) return fail(FT_EINVAL, "bad top-k shape rows=%lld S=%d k=%d", (long long)rows, S, k);
  if (S > 8192 && k > 16384)
    return fail(FT_EUNSUPPORTED, "top-k of rows longer than 8192 takes k <= 16384 (S=%d k=%d)", S, k);
  if (rows > 0x7fffffffLL) return fail(FT_EUNSUPPORTED, "too many rows");
  hipError_t e = ft::launch_topk(score, rows, S, k, idx, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "topk launch");
  return FT_OK;
}

int ft_noise_exp_fill(float* dst, int32_t B, int32_t H, int32_t Sq, int32_t Skv, uint64_t seed, void* stream) {
  if (!dst) return fail(FT_EINVAL, "dst pointer is null");
  if (B < 1 || H < 1 || Sq < 1 || Skv < 1) return fail(FT_EINVAL, "bad shape");
  hipError_t e = ft::launch_noise_fill(dst, B, H, Sq, Skv, seed, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "noise fill launch");
  return FT_OK;
}

int ft_noise_exp_fill_host(float* dst, int32_t B, int32_t H, int32_t Sq, int32_t Skv, uint64_t seed) {
  if (!dst) return fail(FT_EINVAL, "dst pointer is null");
  if (B < 1 || H < 1 || Sq < 1 || Skv < 1) return fail(FT_EINVAL, "bad shape");
  for (int64_t bh = 0; bh < (int64_t)B * H; ++bh) {
    const ft::NoiseKeys nk = ft::noise_keys(seed, (uint32_t)bh);
    for (int i = 0; i < Sq; ++i) {
      const uint32_t a_i = ft::noise_row(nk, (uint32_t)i);
      float* row = dst + (bh * Sq + i) * (int64_t)Skv;
      for (int j = 0; j < Skv; ++j) row[j] = (float)-std::log((double)ft::noise_uniform(a_i, ft::noise_col(nk, (uint32_t)j)));
    }
  }
  return FT_OK;
}

}  // extern "C"
