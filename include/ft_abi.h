/*
 * C ABI of libflashtensor_hip: fused attention-variant kernels for AMD MI355X (gfx950).
 *
 * This is the boundary a host program binds (ctypes, pybind11, cgo ...): plain pointers, sizes and
 * POD structs only.  Every function returns FT_OK (0) or a negative FT_E* code; ft_last_error() then
 * holds a thread-local message.  Device pointers are borrowed for the duration of the call, nothing
 * is retained, no device memory is allocated or freed, and no call synchronises: kernels are queued
 * on the hipStream_t passed as `stream` (NULL = the null stream).
 *
 * What each entry point replaces in the reference (monellz/FlashTensor):
 *   the emitted kernel wrapper `def <Kernel>(arg0: torch.Tensor, ...) -> Tuple[...]` that allocates the
 *   results and launches the fused Triton kernel (lib/Translate/to_triton.cpp:529-638, device kernel
 *   :480-527), and the TensorRT closure used by the harnesses
 *   (python/asuka/backend/tensorrt/builder.py:73-151), for the workloads defined in
 *   cases/kernels/{attn,h2o,kf,roco,snapkv,corm,gemma2}.py and bench/{ea,sima}.mlir.
 */
#ifndef FT_ABI_H
#define FT_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FT_ABI_VERSION 5

enum FtStatus {
  FT_OK = 0,
  FT_EINVAL = -1,       /* bad argument (null pointer, shape, stride, alignment) */
  FT_EUNSUPPORTED = -2, /* valid request the kernels do not cover (head_dim, dtype, ...) */
  FT_ELAUNCH = -3,      /* HIP reported an error at launch */
  FT_EWORKSPACE = -4    /* workspace missing or smaller than ft_workspace_bytes() */
};

enum FtDtype { FT_F16 = 0, FT_BF16 = 1, FT_F32 = 2 };

enum FtFlags {
  FT_CAUSAL = 1u,      /* mask key j for query i when j > i + (Skv - Sq)  (cases/kernels/attn.py:22-23) */
  FT_FAST_LOGITS = 2u  /* keep QK^T/sqrt(D) in fp32 instead of reproducing the reference's fp16 rounding
                          of the logits (cases/kernels/attn.py:29); faster, ~1e-3 relative on probabilities */
};

enum FtOp { FT_OP_ATTN = 0, FT_OP_COLSTATS = 1, FT_OP_KEYFORMER = 2, FT_OP_EA = 3, FT_OP_SIMA = 4, FT_OP_CORM = 5 };

/* Element strides of a logical [B, S, H, D] tensor; the D axis must be contiguous (stride 1). */
typedef struct FtStrides {
  int64_t b, s, h;
} FtStrides;

/* One attention problem: q [B,Sq,H,D], k,v [B,Skv,Hkv,D], o [B,Sq,H,D] (cases/kernels/attn.py:37-39, :32-34).
 * Hkv = 0 or H: one k/v head per query head.  Hkv < H (H a multiple of Hkv): grouped queries as in
 * cases/attn.py:29-31, query head h reads k/v head h / (H / Hkv); sk.h, sv.h are then strides of k/v heads. */
typedef struct FtAttnArgs {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  FtStrides sq, sk, sv, so;
  int32_t B, H, Sq, Skv, D;
  int32_t dtype;  /* FtDtype of q, k, v, o */
  uint32_t flags; /* FtFlags */
  int32_t Hkv;    /* number of k/v heads; 0 means H */
} FtAttnArgs;

/* KeyFormer noise source.  exp_rand != NULL: the reference's input tensor [B,H,Sq,Skv] fp32
 * (cases/kernels/kf.py:19,36-37) with the given element strides (last axis contiguous); every element
 * positive and finite, pairs hidden by the causal mask included: the reference adds -log(exp_rand) to the whole
 * score matrix (kf.py:36-38), and the kernels may read any element of the tensor for a pair they then mask.
 * exp_rand == NULL: drawn in-kernel from the counter-based stream keyed by `seed`
 * (ft_noise_exp_fill* materialise the same tensor).  That stream is this library's own definition (the reference
 * has none: it takes the tensor as an input); it is fixed for a given FT_ABI_VERSION, and a change of the
 * stream changes that version. */
typedef struct FtNoise {
  const float* exp_rand;
  int64_t stride_b, stride_h, stride_row;
  uint64_t seed;
} FtNoise;

int ft_abi_version(void);
const char* ft_last_error(void);

/* Bytes of device scratch the op needs for this problem (0 if none).  The caller owns the buffer. */
size_t ft_workspace_bytes(int op, const FtAttnArgs* a);

/* Causal (or full) softmax attention: replaces the fused kernel of Attn.forward (cases/kernels/attn.py:18-34).
 * lse: optional [B,H,Sq] fp32 output, log2-domain row normaliser max + log2(sum). */
int ft_attn_fwd(const FtAttnArgs* a, float* lse, void* stream);

/* Attention + per-key column statistics: H2O.forward (cases/kernels/h2o.py:18-38; colsumsq == NULL) and
 * RoCo.forward (cases/kernels/roco.py:18-48).  colsum, colsumsq: [B,H,Skv] fp32.
 * Grouped queries (Hkv < H, colsumsq == NULL only): colsum is [B,Hkv,Skv], the column sums of the
 * probabilities averaged over the query heads of each group (cases/attn_h2o.py:42-47). */
int ft_attn_colstats_fwd(const FtAttnArgs* a, float* colsum, float* colsumsq, void* workspace, size_t workspace_bytes,
                         void* stream);

/* ft_attn_colstats_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): no workspace argument; the row normalisers (and the per-head
 * sums of grouped queries) live in a static device buffer of FT_STATIC_SCRATCH_BYTES that the library's code object
 * carries on every GPU it is loaded on.  No counterpart in the reference.  Problems whose
 * ft_workspace_bytes(FT_OP_COLSTATS, a) exceeds the buffer are refused with FT_EWORKSPACE.  Calls no allocator.
 * All calls on one GPU share that GPU's buffer: two calls that overlap in time on one GPU (different streams or
 * threads) race; calls on one stream are ordered.  Results are those of ft_attn_colstats_fwd, bit for bit.
 * The buffer's address is looked up (hipGetSymbolAddress) on the first call on each device: make that first call
 * outside graph capture.  `stream` must belong to the current device (FT_EINVAL otherwise). */
#define FT_STATIC_SCRATCH_BYTES (8u << 20)
int ft_attn_colstats_fwd_static(const FtAttnArgs* a, float* colsum, float* colsumsq, void* stream);

/* KeyFormer.forward (cases/kernels/kf.py:19-42): attention + column sums of softmax((logits + gumbel)/tau),
 * gumbel = -log(exp_rand).  kf_score: [B,H,Skv] fp32. */
int ft_keyformer_fwd(const FtAttnArgs* a, const FtNoise* noise, float tau, float* kf_score, void* workspace,
                     size_t workspace_bytes, void* stream);

/* Gemma2.forward (cases/kernels/gemma2.py:19-39): attention whose scaled logits pass through
 * softcap * tanh(logit / softcap) (three 16-bit tensor ops in the reference, :31-33) before the mask and
 * the softmax.  lse: optional [B,H,Sq] fp32 as for ft_attn_fwd. */
int ft_attn_softcap_fwd(const FtAttnArgs* a, float softcap, float* lse, void* stream);

/* Corm.forward (cases/kernels/corm.py:18-40): attention + corm_score[b,h,j] = any_i(probs[b,h,i,j] >=
 * corm_mask[i,j]) as uint8 [B,H,Skv].  corm_mask: fp32 [Sq,Skv] with the given row stride, thresholds > 0
 * (pairs hidden by the causal mask are not compared); NULL = the reference's own recipe 1 / (i + 1)
 * (corm.py:47-49), evaluated in the log domain without reading a tensor.  A probability within 1e-6
 * (relative) of its threshold counts as reaching it, so the reference's exact ties (p_00 = 1 against 1) are kept.
 * margin: optional [B,H,Skv] fp32 distance from the boundary: max_i log2(p_ij (i + 1)) for the recipe,
 * max_i (p_ij - (1 - 1e-6) mask_ij) for a tensor. */
int ft_corm_fwd(const FtAttnArgs* a, const float* corm_mask, int64_t mask_row_stride, uint8_t* corm_score, float* margin,
                void* workspace, size_t workspace_bytes, void* stream);

/* SnapKV's smoothing of the per-key scores (cases/kernels/snapkv.py:39): dst[r, j] = (1 / kernel) * sum of
 * src[r, j - kernel/2 .. j + kernel/2] with zeros outside the row, kernel odd; src, dst: [rows, S] fp32. */
int ft_avgpool1d(const float* src, int64_t rows, int32_t S, int32_t kernel, float* dst, void* stream);

/* Linear attention cores of bench/ea.mlir:13-17 (kind = FT_OP_EA) and bench/sima.mlir:13-17 (FT_OP_SIMA):
 * O = f(Q) (g(K)^T V).  normalize_q applies SimA's L1 normalisation to Q as well (ignored for EA).
 * a->dtype: FT_F16 or FT_BF16 (the harness's type switch, cases/attn.py:90,97; MFMA operands of that type), or
 * FT_F32, the type of the .mlir functions (ea.mlir:2): fp32 tensors are rounded to fp16 as they are loaded.
 * out_dtype: FtDtype of o, the input type or FT_F32 (FT_F32 only for fp32 inputs).  Strides are multiples of 16
 * bytes.  head_dim 64, or 32 (the .mlir's own 4 heads of 32, :7-9) with an even number of heads stored 32 elements
 * apart (s*.h == 32). */
int ft_linattn_fwd(const FtAttnArgs* a, int kind, int normalize_q, int out_dtype, void* workspace,
                   size_t workspace_bytes, void* stream);

/* The whole block of bench/ea.mlir:2-23 / bench/sima.mlir:2-23 around the core: x [B,S,C] with C = H*D,
 * qkv = x w_qkv^T + b_qkv (w_qkv [3C,C] row-major as in a Linear, :3-5), split into q, k, v and into heads
 * (:6-12), the core (:13-17), y = core w_out^T + b_out (w_out [C,C], :20-22).  All tensors of one type (fp16,
 * bf16, or the .mlir's own fp32) and contiguous; biases may be NULL.  The two projections are hipBLASLt GEMMs (fp32
 * accumulation, bias added before the one rounding to the tensor type); q/k/v and the core's result live in the
 * workspace as tensors of that type.  D = 64, or 32 with an even H.
 * Narrow models (D = 32 with 2 or 4 heads, the .mlir's own geometry; short calls, or batches enough to cover the chip) run as
 * two launches of this library's own instead: projection weights in LDS, q / k / v never leave registers, MFMA
 * operands of the tensor type (fp16 for fp32 tensors: x and the weights are rounded as they are loaded), no
 * hipBLASLt involved. */
typedef struct FtLinBlockArgs {
  const void* x;
  const void* w_qkv;
  const void* b_qkv;
  const void* w_out;
  const void* b_out;
  void* y;
  int32_t B, S, H, D;
  int32_t dtype; /* FtDtype of every tensor */
} FtLinBlockArgs;

/* 0 if the arguments are not supported (ft_last_error() says why). */
size_t ft_linattn_block_workspace_bytes(const FtLinBlockArgs* b, int kind);

/* Where the projections are library GEMMs, hipBLASLt is opened on first use (FT_EUNSUPPORTED if it cannot be found);
 * its handle and the GEMM plans are cached per device and shape, and those calls serialise on one mutex. */
int ft_linattn_block_fwd(const FtLinBlockArgs* b, int kind, int normalize_q, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Heavy hitters: indices of the k largest entries of each row of score [rows, S] fp32, in descending
 * score order (ties: lower index first), written as int64 [rows, k].  Not in the reference, whose H2O
 * case ends at the score (cases/kernels/h2o.py:34-38).  Rows of up to 8192 entries are sorted whole (any k <= S); longer rows take
 * k <= 16384 (a radix select of the k-th score, then a sort of the k winners), FT_EUNSUPPORTED beyond. */
int ft_topk(const float* score, int64_t rows, int32_t S, int32_t k, int64_t* idx, void* stream);

/* The tensor E[B,H,Sq,Skv] = -ln(u) drawn by the seeded KeyFormer mode, written to device memory
 * (ft_noise_exp_fill) or host memory (ft_noise_exp_fill_host). */
int ft_noise_exp_fill(float* dst, int32_t B, int32_t H, int32_t Sq, int32_t Skv, uint64_t seed, void* stream);
int ft_noise_exp_fill_host(float* dst, int32_t B, int32_t H, int32_t Sq, int32_t Skv, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif /* FT_ABI_H */
