// The whole block of bench/ea.mlir / bench/sima.mlir around the linear-attention core: the fused q/k/v
// Linear (ea.mlir:3-5), the split into heads (:6-12, done with strides, nothing is moved), the core
// (:13-17, ft_linattn_fwd) and the output Linear (:20-22).  The two projections are plain library GEMMs
// with a bias epilogue and go to hipBLASLt; the library is opened with dlopen on first use so that the rest
// of this library neither links against it nor needs it.
#include <dlfcn.h>
#include <stdlib.h>
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "../../include/ft_abi.h"

namespace ft {
int set_error(int code, const char* fmt, ...);
// linblock_small.hip: the two-launch form for heads of 32 channels and C <= 128
void small_block_plan(const FtLinBlockArgs& a, int* nch, int* strips_per_chunk);
size_t small_block_workspace_bytes(const FtLinBlockArgs& a);
hipError_t launch_small_block(const FtLinBlockArgs& a, int kind, int normalize_q, void* ws, hipStream_t s);
}

namespace {

constexpr size_t kLtWorkspace = 32u << 20;  // scratch offered to hipBLASLt's kernels (split-k and the like)

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

struct LtApi {
  void* lib = nullptr;
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  const char* missing = nullptr;
};

template <class F>
bool bind(LtApi& api, F& fn, const char* name) {
  fn = reinterpret_cast<F>(dlsym(api.lib, name));
  if (!fn && !api.missing) api.missing = name;
  return fn != nullptr;
}

LtApi& lt_api() {
  static LtApi api;
  static std::once_flag once;
  std::call_once(once, [] {
    // a copy the process already holds (the one torch ships, say) is preferred over loading a second one
    const char* names[] = {"libhipblaslt.so.1", "libhipblaslt.so", "/opt/rocm/lib/libhipblaslt.so.1"};
    for (const char* n : names)
      if ((api.lib = dlopen(n, RTLD_NOW | RTLD_LOCAL | RTLD_NOLOAD))) break;
    if (!api.lib)
      for (const char* n : names)
        if ((api.lib = dlopen(n, RTLD_NOW | RTLD_LOCAL))) break;
    if (!api.lib) {
      api.missing = "libhipblaslt.so.1";
      return;
    }
    bind(api, api.create, "hipblasLtCreate");
    bind(api, api.layout_create, "hipblasLtMatrixLayoutCreate");
    bind(api, api.desc_create, "hipblasLtMatmulDescCreate");
    bind(api, api.desc_set, "hipblasLtMatmulDescSetAttribute");
    bind(api, api.pref_create, "hipblasLtMatmulPreferenceCreate");
    bind(api, api.pref_set, "hipblasLtMatmulPreferenceSetAttribute");
    bind(api, api.pref_destroy, "hipblasLtMatmulPreferenceDestroy");
    bind(api, api.heuristic, "hipblasLtMatmulAlgoGetHeuristic");
    bind(api, api.matmul, "hipblasLtMatmul");
  });
  return api;
}

// One Linear: y[M,N] = x[M,K] w[N,K]^T + bias[N], all row-major and of one type (fp16, bf16 or fp32), fp32 accumulation.  In the
// column-major terms of the library: D[N,M] = op_T(A = w as [K,N]) * (B = x as [K,M]), bias along D's rows.
struct LinearPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

struct LtState {
  std::mutex mu;
  std::map<int, hipblasLtHandle_t> handles;                               // per device
  std::map<std::tuple<int, int64_t, int64_t, int64_t, bool, int>, LinearPlan> plans;  // (device, M, N, K, bias, dtype)
};

LtState& lt_state() {
  static LtState s;
  return s;
}

#define LT_TRY(call, what)                                                                         \
  do {                                                                                             \
    hipblasStatus_t st__ = (call);                                                                 \
    if (st__ != HIPBLAS_STATUS_SUCCESS) return ft::set_error(FT_ELAUNCH, "hipBLASLt %s failed with status %d", what, (int)st__); \
  } while (0)

// Callers hold LtState::mu.
int linear(LtApi& api, LtState& st, int device, int dtype, const void* x, const void* w, const void* bias, void* y, int64_t M,
           int64_t N, int64_t K, void* lt_ws, hipStream_t stream) {
  const hipDataType lt_type = dtype == FT_F32 ? HIP_R_32F : dtype == FT_BF16 ? HIP_R_16BF : HIP_R_16F;
  hipblasLtHandle_t handle;
  auto hit = st.handles.find(device);
  if (hit == st.handles.end()) {
    LT_TRY(api.create(&handle), "handle creation");
    st.handles[device] = handle;
  } else {
    handle = hit->second;
  }
  const auto key = std::make_tuple(device, M, N, K, bias != nullptr, dtype);
  auto pit = st.plans.find(key);
  if (pit == st.plans.end()) {
    LinearPlan p;
    LT_TRY(api.desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "descriptor creation");
    const int32_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    LT_TRY(api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)), "transA");
    LT_TRY(api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)), "transB");
    if (bias) {
      const uint32_t epi = HIPBLASLT_EPILOGUE_BIAS;
      const int32_t bias_type = lt_type;
      LT_TRY(api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi)), "epilogue");
      LT_TRY(api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)), "bias type");
      // the heuristic wants a bias pointer in place; the real one is set before every call
      LT_TRY(api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)), "bias pointer");
    }
    LT_TRY(api.layout_create(&p.a, lt_type, (uint64_t)K, (uint64_t)N, K), "layout A");
    LT_TRY(api.layout_create(&p.b, lt_type, (uint64_t)K, (uint64_t)M, K), "layout B");
    LT_TRY(api.layout_create(&p.d, lt_type, (uint64_t)N, (uint64_t)M, N), "layout D");
    hipblasLtMatmulPreference_t pref;
    LT_TRY(api.pref_create(&pref), "preference creation");
    const uint64_t max_ws = kLtWorkspace;
    LT_TRY(api.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws)), "workspace preference");
    hipblasLtMatmulHeuristicResult_t res[1];
    int found = 0;
    hipblasStatus_t hs = api.heuristic(handle, p.desc, p.a, p.b, p.d, p.d, pref, 1, res, &found);
    api.pref_destroy(pref);
    if (hs != HIPBLAS_STATUS_SUCCESS || found < 1)
      return ft::set_error(FT_EUNSUPPORTED, "hipBLASLt has no kernel for a %lld x %lld x %lld Linear of dtype %d (status %d)",
                           (long long)M, (long long)N, (long long)K, dtype, (int)hs);
    p.algo = res[0].algo;
    p.workspace = res[0].workspaceSize;
    pit = st.plans.emplace(key, p).first;
  }
  LinearPlan& p = pit->second;
  if (bias) LT_TRY(api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)), "bias pointer");
  const float one = 1.f, zero = 0.f;
  LT_TRY(api.matmul(handle, p.desc, &one, w, p.a, x, p.b, &zero, y, p.d, y, p.d, &p.algo, lt_ws, p.workspace, stream),
         "matmul");
  return FT_OK;
}

int check_block(const FtLinBlockArgs* b, int kind) {
  if (!b) return ft::set_error(FT_EINVAL, "args is null");
  if (kind != FT_OP_EA && kind != FT_OP_SIMA) return ft::set_error(FT_EINVAL, "kind must be FT_OP_EA or FT_OP_SIMA");
  if (b->B < 1 || b->S < 1 || b->H < 1) return ft::set_error(FT_EINVAL, "bad shape B=%d S=%d H=%d", b->B, b->S, b->H);
  if (b->D != 64 && !(b->D == 32 && (b->H & 1) == 0))
    return ft::set_error(FT_EUNSUPPORTED, "head_dim %d with %d heads not supported by the linear-attention kernels (64, or 32 with an even number of heads)", b->D, b->H);
  if (b->dtype != FT_F16 && b->dtype != FT_BF16 && b->dtype != FT_F32)
    return ft::set_error(FT_EUNSUPPORTED, "dtype %d not supported by the linear-attention kernels (f16, bf16 or f32)", b->dtype);
  return FT_OK;
}

struct BlockLayout {
  size_t qkv, core, lin, lt, total;
  FtAttnArgs a;
};

BlockLayout block_layout(const FtLinBlockArgs& b, int kind, char* base) {
  BlockLayout l;
  const int64_t C = (int64_t)b.H * b.D;
  const size_t tokens = (size_t)b.B * b.S;
  const size_t es = b.dtype == FT_F32 ? 4 : 2;
  l.qkv = 0;
  l.core = l.qkv + align256(tokens * 3 * C * es);
  l.lin = l.core + align256(tokens * C * es);
  FtAttnArgs a{};
  a.q = base + l.qkv;
  a.k = base + l.qkv + C * es;
  a.v = base + l.qkv + 2 * C * es;
  a.o = base + l.core;
  a.sq = a.sk = a.sv = FtStrides{(int64_t)b.S * 3 * C, 3 * C, b.D};
  a.so = FtStrides{(int64_t)b.S * C, C, b.D};
  a.B = b.B;
  a.H = b.H;
  a.Sq = a.Skv = b.S;
  a.D = b.D;
  a.dtype = b.dtype;
  l.a = a;
  l.lt = l.lin + align256(ft_workspace_bytes(kind, &a));
  l.total = l.lt + kLtWorkspace;
  // the two-launch form of narrow models keeps its per-chunk partial matrices there instead (0 where it does not apply)
  const size_t small = ft::small_block_workspace_bytes(b);
  if (small > l.total) l.total = small;
  return l;
}

}  // namespace

extern "C" {

size_t ft_linattn_block_workspace_bytes(const FtLinBlockArgs* b, int kind) {
  if (check_block(b, kind) != FT_OK) return 0;
  return block_layout(*b, kind, nullptr).total;
}

int ft_linattn_block_fwd(const FtLinBlockArgs* b, int kind, int normalize_q, void* workspace, size_t workspace_bytes,
                         void* stream) {
  int rc = check_block(b, kind);
  if (rc != FT_OK) return rc;
  if (!b->x || !b->w_qkv || !b->w_out || !b->y) return ft::set_error(FT_EINVAL, "x / w_qkv / w_out / y pointer is null");
  const uintptr_t ptrs = (uintptr_t)b->x | (uintptr_t)b->w_qkv | (uintptr_t)b->w_out | (uintptr_t)b->y |
                         (uintptr_t)b->b_qkv | (uintptr_t)b->b_out | (uintptr_t)workspace;
  if (ptrs & 15) return ft::set_error(FT_EINVAL, "x, weights, biases, y and the workspace must be 16-byte aligned");
  BlockLayout l = block_layout(*b, kind, static_cast<char*>(workspace));
  if (!workspace || workspace_bytes < l.total)
    return ft::set_error(FT_EWORKSPACE, "workspace of %zu bytes needed, got %zu", l.total, workspace ? workspace_bytes : (size_t)0);
  {
    // narrow models (the .mlir's own 4 heads of 32): weights in LDS, q / k / v in registers, two launches.
    // FT_LINBLOCK_FORM=gemm in the environment is a test hook that keeps the library-GEMM form for them.
    int nch = 0, spc = 0;
    ft::small_block_plan(*b, &nch, &spc);
    const char* form = getenv("FT_LINBLOCK_FORM");
    if (nch > 0 && ft::small_block_workspace_bytes(*b) <= workspace_bytes && !(form && form[0] == 'g')) {
      hipError_t le = ft::launch_small_block(*b, kind, normalize_q, workspace, (hipStream_t)stream);
      if (le != hipSuccess) return ft::set_error(FT_ELAUNCH, "linear block launch: %s", hipGetErrorString(le));
      return FT_OK;
    }
  }
  LtApi& api = lt_api();
  if (api.missing) return ft::set_error(FT_EUNSUPPORTED, "hipBLASLt is not available (%s not found)", api.missing);
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return ft::set_error(FT_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));

  char* base = static_cast<char*>(workspace);
  const int64_t C = (int64_t)b->H * b->D, M = (int64_t)b->B * b->S;
  LtState& st = lt_state();
  std::lock_guard<std::mutex> lock(st.mu);
  rc = linear(api, st, device, b->dtype, b->x, b->w_qkv, b->b_qkv, base + l.qkv, M, 3 * C, C, base + l.lt, (hipStream_t)stream);
  if (rc != FT_OK) return rc;
  rc = ft_linattn_fwd(&l.a, kind, normalize_q, b->dtype, base + l.lin, l.lt - l.lin, stream);
  if (rc != FT_OK) return rc;
  return linear(api, st, device, b->dtype, base + l.core, b->w_out, b->b_out, b->y, M, C, C, base + l.lt, (hipStream_t)stream);
}

}  // extern "C"
