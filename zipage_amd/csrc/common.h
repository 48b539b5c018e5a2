// Shared device/host helpers for the KV-compression kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/zipage_hip.h"

#define ZP_WAVE 64

// ---------------------------------------------------------------- error reporting
void zp_set_error(const char* fmt, ...);

#define ZP_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      zp_set_error(__VA_ARGS__);         \
      return ZP_EINVAL;                  \
    }                                    \
  } while (0)

#define ZP_LAUNCH_CHECK()                                              \
  do {                                                                 \
    hipError_t e_ = hipGetLastError();                                 \
    if (e_ != hipSuccess) {                                            \
      zp_set_error("%s:%d HIP launch failed: %s", __FILE__, __LINE__,  \
                   hipGetErrorString(e_));                             \
      return ZP_EHIP;                                                  \
    }                                                                  \
  } while (0)

// The scratch the one-sweep scorer of one cache dtype asks for (declared in the header too).
extern "C" int64_t zp_attention_score_workspace_for(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                                    int32_t Hkv, int32_t Hq, int32_t W, int32_t dtype);
// Scratch zp_attention_score cannot do without (it takes the three-sweep kernel when the caller
// brings less than zp_attention_score_workspace() asks for).  Library-internal.
int64_t zp_attention_score_workspace_floor(int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                                           int32_t Hq, int32_t W);
// gather.hip, library-internal: K/V compaction and the carried scores' compaction in one launch
// where the shapes allow it (zp_compress_kv followed by zp_compress_score otherwise); the
// arguments of the two.
int zp_compress_kv_and_score(void* key, void* value, void* score_cache, const void* scores_src,
                             const uint8_t* flag, const int32_t* block_table,
                             const int32_t* target_block_table, int32_t L, int32_t B, int32_t NB,
                             int32_t BS, int32_t Hkv, int32_t D, int32_t num_pages,
                             int32_t target_width, int64_t k_sl, int64_t k_sp, int64_t k_ss,
                             int64_t k_sh, int64_t v_sl, int64_t v_sp, int64_t v_ss, int64_t v_sh,
                             int64_t c_sl, int64_t c_sp, int64_t c_ss, int64_t c_sh, int32_t dtype,
                             void* stream);

// ---------------------------------------------------------------- element types
// Storage element tags.  bf16/fp16 are kept as raw 16-bit patterns in memory.
struct BF16 { typedef uint16_t raw; static constexpr int bytes = 2; };
struct F16  { typedef uint16_t raw; static constexpr int bytes = 2; };
struct F32  { typedef float raw;    static constexpr int bytes = 4; };

__device__ __forceinline__ float bf16_bits_to_float(uint16_t h) {
  return __uint_as_float(((uint32_t)h) << 16);
}
// Round-to-nearest-even, infinities preserved, NaN kept quiet: the hardware conversion
// (v_cvt_pk_bf16_f32), one instruction.
typedef float zp_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 zp_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  const zp_f32x2 v = {f, 0.f};
  return (uint16_t)__builtin_bit_cast(uint32_t, __builtin_convertvector(v, zp_bf16x2));
}
// The rounded value as fp32: with the value in the high half of the packed result and a zero in
// the low half, the 32-bit result is the answer.
__device__ __forceinline__ float bf16_round(float f) {
  const zp_f32x2 v = {0.f, f};
  return __builtin_bit_cast(float, __builtin_convertvector(v, zp_bf16x2));
}
__device__ __forceinline__ float f16_bits_to_float(uint16_t h) {
  union { uint16_t u; _Float16 f; } c; c.u = h; return (float)c.f;
}
__device__ __forceinline__ uint16_t float_to_f16_bits(float f) {
  union { uint16_t u; _Float16 f; } c; c.f = (_Float16)f; return c.u;
}

template <typename T> struct Elem;
template <> struct Elem<BF16> {
  __device__ static __forceinline__ float ld(const void* p, int64_t i) { return bf16_bits_to_float(((const uint16_t*)p)[i]); }
  __device__ static __forceinline__ void st(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = float_to_bf16_bits(v); }
  __device__ static __forceinline__ float rnd(float v) { return bf16_round(v); }
};
template <> struct Elem<F16> {
  __device__ static __forceinline__ float ld(const void* p, int64_t i) { return f16_bits_to_float(((const uint16_t*)p)[i]); }
  __device__ static __forceinline__ void st(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = float_to_f16_bits(v); }
  __device__ static __forceinline__ float rnd(float v) { return f16_bits_to_float(float_to_f16_bits(v)); }
};
template <> struct Elem<F32> {
  __device__ static __forceinline__ float ld(const void* p, int64_t i) { return ((const float*)p)[i]; }
  __device__ static __forceinline__ void st(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
  __device__ static __forceinline__ float rnd(float v) { return v; }
};

// Dispatch a templated launcher on the runtime dtype tag.
#define ZP_DISPATCH_DTYPE(dtype, ...)                                   \
  switch (dtype) {                                                      \
    case ZP_BF16: { typedef BF16 T; __VA_ARGS__; } break;               \
    case ZP_F16:  { typedef F16 T;  __VA_ARGS__; } break;               \
    case ZP_F32:  { typedef F32 T;  __VA_ARGS__; } break;               \
    default: zp_set_error("unknown dtype tag %d", (int)(dtype)); return ZP_EINVAL; \
  }

static inline int zp_dtype_bytes(int dtype) { return dtype == ZP_F32 ? 4 : 2; }

// ---------------------------------------------------------------- page-table codes
// id >= 0: full page; -1: padding; x < -1: the sequence's last page, id = -x-2.
__device__ __forceinline__ bool page_is_pad(int code) { return code == -1; }
__device__ __forceinline__ bool page_is_last(int code) { return code < -1; }
__device__ __forceinline__ int page_id(int code) { return code < -1 ? -code - 2 : code; }

// ---------------------------------------------------------------- wave helpers
// Cross-lane exchanges without the LDS crossbar: DPP rotations inside a row of 16 lanes, and the
// gfx950 lane-swap instructions for the two wider steps.  A ds_bpermute round trip costs a
// hundred-odd cycles of latency; these are ordinary VALU instructions.
template <int N> __device__ __forceinline__ int dpp_row_ror(int x) {
  return __builtin_amdgcn_update_dpp(0, x, 0x120 + N, 0xf, 0xf, false);  // lane i <- lane (i-N)%16 of its row
}
// lane i <- lane i+N of its row of 16 (0 where that lane lies outside the row)
template <int N> __device__ __forceinline__ float dpp_row_shl(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x100 + N, 0xf, 0xf, false));
}
template <int N> __device__ __forceinline__ float dpp_row_ror(float x) {
  return __builtin_bit_cast(float, dpp_row_ror<N>(__builtin_bit_cast(int, x)));
}
// value of lane ^ 16 (v_permlane16_swap: odd rows of one operand <-> even rows of the other)
__device__ __forceinline__ int lane_xor16(int x) {
  const auto r = __builtin_amdgcn_permlane16_swap((unsigned)x, (unsigned)x, false, false);
  return (int)((threadIdx.x & 16) ? r[0] : r[1]);
}
__device__ __forceinline__ float lane_xor16(float x) {
  return __builtin_bit_cast(float, lane_xor16(__builtin_bit_cast(int, x)));
}
// value of lane ^ 32 (v_permlane32_swap: upper half of one operand <-> lower half of the other)
__device__ __forceinline__ int lane_xor32(int x) {
  const auto r = __builtin_amdgcn_permlane32_swap((unsigned)x, (unsigned)x, false, false);
  return (int)((threadIdx.x & 32) ? r[0] : r[1]);
}
__device__ __forceinline__ float lane_xor32(float x) {
  return __builtin_bit_cast(float, lane_xor32(__builtin_bit_cast(int, x)));
}
// all-reduce over the 16 lanes of a row (every lane ends with the result)
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_row_ror<8>(v);
  v += dpp_row_ror<4>(v);
  v += dpp_row_ror<2>(v);
  v += dpp_row_ror<1>(v);
  return v;
}
__device__ __forceinline__ int row16_sum(int v) {
  v += dpp_row_ror<8>(v);
  v += dpp_row_ror<4>(v);
  v += dpp_row_ror<2>(v);
  v += dpp_row_ror<1>(v);
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_row_ror<8>(v));
  v = fmaxf(v, dpp_row_ror<4>(v));
  v = fmaxf(v, dpp_row_ror<2>(v));
  v = fmaxf(v, dpp_row_ror<1>(v));
  return v;
}
// all-reduce over 32 lanes (each half of the wave separately) and over the whole wave
__device__ __forceinline__ float half_sum(float v) { v = row16_sum(v); return v + lane_xor16(v); }
__device__ __forceinline__ float half_max(float v) { v = row16_max(v); return fmaxf(v, lane_xor16(v)); }
__device__ __forceinline__ float wave_max(float v) { v = half_max(v); return fmaxf(v, lane_xor32(v)); }
__device__ __forceinline__ float wave_sum(float v) { v = half_sum(v); return v + lane_xor32(v); }
__device__ __forceinline__ int wave_sum_i(int v) {
  v = row16_sum(v);
  v += lane_xor16(v);
  return v + lane_xor32(v);
}
// Inclusive prefix sum over the 64 lanes of a wave in six DPP adds: shifts by 1, 2, 4 and 8 inside
// each row of 16 lanes (lanes without a source add 0), then lane 15 of rows 0 / 2 is added to rows
// 1 / 3 and lane 31 to the upper half.
__device__ __forceinline__ int wave_prefix_sum_incl(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 -> rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 -> rows 2, 3
  return v;
}
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }
__device__ __forceinline__ uint64_t lanemask_lt() {
  return (1ull << lane_id()) - 1ull;
}

struct __attribute__((aligned(16))) vec16 { uint32_t x, y, z, w; };
