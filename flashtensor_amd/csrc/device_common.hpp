// Device-side building blocks shared by the gfx950 kernels: MFMA operand types, LDS tile staging with
// XOR swizzles, transposed LDS reads, wave-level exchanges.
//
// MFMA operand layouts used throughout (v_mfma_f32_32x32x16_{f16,bf16}, wave64), lane l, g = l / 32:
//   A (32 x 16): lane holds row l % 32, k = 8 g + [0..7]
//   B (16 x 32): lane holds column l % 32, k = 8 g + [0..7]
//   C (32 x 32): lane holds column l % 32, register r holds row 8 (r / 4) + 4 g + r % 4
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ft {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

#define FT_LDS(T, p) ((__attribute__((address_space(3))) T*)(p))

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Element traits: 16-bit storage type <-> MFMA flavour.
struct F16 {
  typedef half8 vec8;
  typedef _Float16 elem;
  static __device__ __forceinline__ elem to_elem(uint16_t bits) { return __builtin_bit_cast(_Float16, bits); }
  static __device__ __forceinline__ float16v mfma(vec8 a, vec8 b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  // 16x16x32: lane l holds row (A) / column (B) l % 16 and contraction slots 8 (l / 16) + [0..7]; of the result,
  // column l % 16 and rows 4 (l / 16) + [0..3]
  static __device__ __forceinline__ float4v mfma16(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_float(float x) {
    _Float16 h = (_Float16)x;
    return __builtin_bit_cast(uint16_t, h);
  }
  static __device__ __forceinline__ float to_float(uint16_t x) { return (float)__builtin_bit_cast(_Float16, x); }
  // two floats rounded to the storage type in one 32-bit word; its halves as floats; acc + lo + hi
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    const float2v v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, half2v));
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(half2v, w)[0]; }
  static __device__ __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(half2v, w)[1]; }
  static __device__ __forceinline__ float add2(uint32_t w, float acc) {
    const half2v ones = {(_Float16)1.f, (_Float16)1.f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, w), ones, acc, false);
  }
};
struct BF16 {
  typedef bf16x8 vec8;
  typedef __bf16 elem;
  static __device__ __forceinline__ elem to_elem(uint16_t bits) { return __builtin_bit_cast(__bf16, bits); }
  static __device__ __forceinline__ float16v mfma(vec8 a, vec8 b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float4v mfma16(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_float(float x) {  // round to nearest even (v_cvt_pk_bf16_f32)
    return __builtin_bit_cast(uint16_t, (__bf16)x);
  }
  static __device__ __forceinline__ float to_float(uint16_t x) { return __builtin_bit_cast(float, (uint32_t)x << 16); }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    const float2v v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
  static __device__ __forceinline__ float add2(uint32_t w, float acc) {
    const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), ones, acc, false);
  }
};

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }

// Value held by the partner lane l ^ 32 (the other 16 rows of a 32x32 accumulator column).
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second:
// called with (x, x) it returns {x[0..31], x[0..31]} and {x[32..63], x[32..63]}; every lane then holds
// both values of its pair.  One VALU instruction instead of an LDS round trip.
__device__ __forceinline__ float xchg32(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t lo = r[0], hi = r[1];
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? lo : hi);
#else
  return x;
#endif
}

// max of three, written so that the compiler sees it: it then inserts the wait states a vector instruction needs
// after the matrix instruction whose result it reads (it inserts none around inline assembly).  Selected as
// v_max3_f32 only in translation units built with -fno-honor-nans (the attention kernels): otherwise every fmaxf on
// an MFMA result costs a NaN-quieting move per operand.
__device__ __forceinline__ float max3(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }

// tanh to fp32 accuracy without a hardware instruction: odd polynomial where 1 - 2 / (e^2y + 1) would
// cancel (|y| < 0.25, truncation error < 4e-7 relative), the exponential form elsewhere.
__device__ __forceinline__ float tanh_f32(float y) {
  const float a = __builtin_fabsf(y);
  const float y2 = y * y;
  const float poly = y * (1.f + y2 * (-1.f / 3.f + y2 * (2.f / 15.f + y2 * (-17.f / 315.f + y2 * (62.f / 2835.f)))));
  const float e = __builtin_amdgcn_exp2f(a * (2.f * kLog2e));
  const float big = __builtin_copysignf(1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f), y);
  return a < 0.25f ? poly : big;
}

// tanh as 1 - 2 / (e^2y + 1) for either sign: absolute error ~1e-7 (cancellation for small |y|), which is
// enough where the result is rounded to 16 bits or only shifts a logit by that much; four instructions.
__device__ __forceinline__ float tanh_exp_form(float y) {
  return __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(y * (2.f * kLog2e)) + 1.f), 1.f);
}

__device__ __forceinline__ void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0)

// Orders one wave's LDS traffic for the compiler (a wave-private tile written by some lanes and read by others); the
// hardware already executes a wave's LDS instructions in order.
__device__ __forceinline__ void wave_lds_order() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// ---------------------------------------------------------------------------------------------------
// A tile of ROWS x D 16-bit elements staged in LDS, rows of RB = 2 D bytes split in 16-byte chunks.
// Two placements of chunk c of row r:
//   kRowSwizzle : chunk index ^ ((r / RPW) % CPR)        -> conflict-free 16-byte reads of one chunk
//                 column by 16 consecutive rows (MFMA operand with the contraction axis contiguous)
//   kTrSwizzle  : chunk index ^ (((r / RPW) % GPR) << 2) -> conflict-free ds_read_b64_tr_b16 of 4
//                 consecutive rows x 64 bytes (MFMA operand with the contraction axis strided)
// RPW = rows per 256-byte bank window, CPR = chunks per row, GPR = 64-byte granules per row.
template <int D>
struct TileGeom {
  static constexpr int RB = 2 * D;
  static constexpr int CPR = RB / 16;
  static constexpr int RPW = 256 / RB;
  static constexpr int GPR = RB / 64;
  static __device__ __forceinline__ int row_swz(int r) { return (r / RPW) % CPR; }
  static __device__ __forceinline__ int tr_swz(int r) { return ((r / RPW) % GPR) << 2; }
};

enum Swizzle { kRowSwizzle = 0, kTrSwizzle = 1 };

// Cooperative global -> LDS copy of ROWS x D tiles by NT threads with direct-to-LDS buffer loads
// (buffer_load_dwordx4 ... lds: LDS address = wave-uniform base + lane * 16; the MUBUF form, unlike the
// global_load form, does not make the compiler treat every later LDS wait as a full drain).  The swizzle
// is applied on the global side: the lane that fills LDS slot (r, c') fetches global chunk c' ^ swz(r).
// Per-lane byte offsets are computed once; a tile then costs one load per round with a scalar tile offset.
// Rows >= rows_valid re-read the last valid row (callers mask them).  Completion: wait_vmem() then a
// workgroup barrier.  All byte offsets from `base` must fit in 31 bits (checked by the host).
// The host pass only parses kernel bodies (to emit launch stubs); the buffer-resource type and builtins
// exist in the device pass only.
#if defined(__HIP_DEVICE_COMPILE__)
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ void load_lds16(rsrc_t rsrc, char* lds_dst, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, FT_LDS(void, lds_dst), 16, voff, soff, 0, 0);
}
#else
typedef int rsrc_t;
__device__ inline rsrc_t make_rsrc(const void*) { return 0; }
__device__ inline void load_lds16(rsrc_t, char*, uint32_t, uint32_t) {}
#endif

template <int D, int ROWS, int NT, int SWZ>
struct TileStager {
  typedef TileGeom<D> G;
  static constexpr int ROUNDS = ROWS * G::CPR / NT;
  static_assert((ROWS * G::CPR) % NT == 0, "tile must be a whole number of rounds");
  rsrc_t rsrc;
  uint32_t off[ROUNDS];
  uint32_t row_bytes;

  __device__ __forceinline__ void init(const uint16_t* base, int64_t row_stride) {
    rsrc = make_rsrc(base);
    row_bytes = (uint32_t)(row_stride * 2);
    const int lane = lane_id();
    const int wave = wave_id();
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) {
      const int slot = it * NT + wave * 64 + lane;
      const int r = slot / G::CPR;
      const int cs = slot % G::CPR;
      const int c = cs ^ (SWZ == kRowSwizzle ? G::row_swz(r) : G::tr_swz(r));
      off[it] = (uint32_t)r * row_bytes + c * 16;
    }
  }

  // A tile known to lie entirely inside the operand: straight-line code (one load per round) that a
  // caller can spread between other instructions.
  __device__ __forceinline__ void issue_full(int row0, char* lds_tile) const {
    const int wave = wave_id();
    const uint32_t tile_off = (uint32_t)row0 * row_bytes;  // wave-uniform
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) {
      char* dst = lds_tile + (it * NT + wave * 64) * 16;
      load_lds16(rsrc, dst, off[it], tile_off);
    }
  }

  // Tile whose row 0 is row `row0` of the operand.
  __device__ __forceinline__ void issue(int row0, int rows_valid, char* lds_tile) const {
    const int wave = wave_id();
    const uint32_t tile_off = (uint32_t)row0 * row_bytes;  // wave-uniform
    if (rows_valid >= ROWS) {
      issue_full(row0, lds_tile);
    } else {
      const int lane = lane_id();
#pragma unroll
      for (int it = 0; it < ROUNDS; ++it) {
        const int slot = it * NT + wave * 64 + lane;
        const int r = slot / G::CPR;
        const int cs = slot % G::CPR;
        const int c = cs ^ (SWZ == kRowSwizzle ? G::row_swz(r) : G::tr_swz(r));
        const int rr = r < rows_valid ? r : rows_valid - 1;
        char* dst = lds_tile + (it * NT + wave * 64) * 16;
        load_lds16(rsrc, dst, (uint32_t)rr * row_bytes + c * 16, tile_off);
      }
    }
  }
};

// 8 contiguous elements (one 16-byte chunk `c`) of row `r` from a kRowSwizzle tile.
template <int D, typename V8>
__device__ __forceinline__ V8 read_row_chunk(const char* lds_tile, int r, int c) {
  typedef TileGeom<D> G;
  return *reinterpret_cast<const V8*>(lds_tile + r * G::RB + ((c ^ G::row_swz(r)) << 4));
}

// Transposed operand from a kTrSwizzle tile: the calling lane (column d = d_base + l % 32 of the tile,
// g = l / 32) receives rows {k0 + 4 g + [0..3], k0 + 8 + 4 g + [0..3]} of that column: the 8
// contraction slots that pair with registers [rb .. rb+7] of a 32x32 accumulator whose rows start at k0.
// ds_read_b64_tr_b16: within each 16-lane group, lane i receives element i % 4 of the 8-byte rows
// addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4.
template <int D, typename V8>
__device__ __forceinline__ V8 read_tr_operand(const char* lds_tile, int k0, int d_base) {
  typedef TileGeom<D> G;
  const int l = lane_id();
  const int j16 = l & 15;
  const int dhalf = (l >> 4) & 1;
  const int g = l >> 5;
  const int d0 = d_base + 16 * dhalf + 4 * (j16 & 3);
  const int r0 = k0 + 4 * g + (j16 >> 2);
  const int r1 = r0 + 8;
  const int c = d0 >> 3;
  const int within = (d0 & 7) * 2;
  const char* p0 = lds_tile + r0 * G::RB + ((c ^ G::tr_swz(r0)) << 4) + within;
  const char* p1 = lds_tile + r1 * G::RB + ((c ^ G::tr_swz(r1)) << 4) + within;
  short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(FT_LDS(short4v, p0));
  short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(FT_LDS(short4v, p1));
  short8v both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V8, both);
}

}  // namespace ft
