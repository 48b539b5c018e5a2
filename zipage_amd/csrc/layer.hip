// Fused elementwise pieces of the decoder layer that sit between the GEMMs and the cache
// kernels: residual add + RMSNorm, SiLU-gate multiply, and per-head q/k RMSNorm + rotary
// embedding with the K/V scatter and the window-query capture folded in.  All are one pass over
// their rows (HBM- or launch-bound); the intermediate roundings to the 16-bit dtype follow the
// unfused module sequence so the fused step returns what the separate modules would.
#include "common.h"
#include <math.h>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ void unpack8(const u32x4& v, float* o);
template <> __device__ __forceinline__ void unpack8<BF16>(const u32x4& v, float* o) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(v[i] << 16);
    o[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
  }
}
template <> __device__ __forceinline__ void unpack8<F16>(const u32x4& v, float* o) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = f16_bits_to_float((uint16_t)(v[i] & 0xffffu));
    o[2 * i + 1] = f16_bits_to_float((uint16_t)(v[i] >> 16));
  }
}
template <typename T> __device__ __forceinline__ uint16_t to_bits(float f);
template <> __device__ __forceinline__ uint16_t to_bits<BF16>(float f) { return float_to_bf16_bits(f); }
template <> __device__ __forceinline__ uint16_t to_bits<F16>(float f) { return float_to_f16_bits(f); }
template <typename T> __device__ __forceinline__ u32x4 pack8(const float* o) {
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    v[i] = (uint32_t)to_bits<T>(o[2 * i]) | ((uint32_t)to_bits<T>(o[2 * i + 1]) << 16);
  return v;
}

// ------------------------------------------------------------------ residual add + RMSNorm
// One workgroup per row; a row of up to 8 * kThreads * kMaxPieces elements lives in registers.
constexpr int kMaxPieces = 4;   // hidden <= 8192

template <typename T, bool ADD>
__global__ __launch_bounds__(kThreads) void add_rms_kernel(
    const char* __restrict__ x, char* __restrict__ resid, const char* __restrict__ w,
    char* __restrict__ out, int H, int64_t x_st, int64_t r_st, int64_t o_st, float eps) {
  __shared__ float red[kWaves];
  const int tid = threadIdx.x, row = blockIdx.x;
  const int pieces = H / 8;
  float v[kMaxPieces][8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kMaxPieces; ++k) {
    const int pc = tid + k * kThreads;
    if (pc < pieces) {
      unpack8<T>(*(const u32x4*)(x + row * x_st + pc * 16), v[k]);
      if (ADD) {
        float r[8];
        unpack8<T>(*(const u32x4*)(resid + row * r_st + pc * 16), r);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[k][i] += r[i];
        // the sum rounded to the storage dtype is the new residual; the norm uses the fp32 sum
        *(u32x4*)(resid + row * r_st + pc * 16) = pack8<T>(v[k]);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[k][i] * v[k][i];
    }
  }
  ss = wave_sum(ss);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) tot += red[i];
  const float rs = rsqrtf(tot / (float)H + eps);
#pragma unroll
  for (int k = 0; k < kMaxPieces; ++k) {
    const int pc = tid + k * kThreads;
    if (pc < pieces) {
      float wv[8], o[8];
      unpack8<T>(*(const u32x4*)(w + pc * 16), wv);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = Elem<T>::rnd(v[k][i] * rs) * wv[i];
      *(u32x4*)(out + row * o_st + pc * 16) = pack8<T>(o);
    }
  }
}

// ------------------------------------------------------------------ silu(gate) * up
template <typename T>
__global__ __launch_bounds__(kThreads) void silu_mul_kernel(
    const char* __restrict__ gu, char* __restrict__ out, int pieces_per_row, int64_t total_pieces,
    int64_t gu_st, int64_t o_st, int64_t up_off) {
  const int64_t id = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (id >= total_pieces) return;
  const int64_t row = id / pieces_per_row, pc = id - row * pieces_per_row;
  float g[8], u[8], o[8];
  unpack8<T>(*(const u32x4*)(gu + row * gu_st + pc * 16), g);
  unpack8<T>(*(const u32x4*)(gu + row * gu_st + up_off + pc * 16), u);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = Elem<T>::rnd(g[i] / (1.f + __expf(-g[i]))) * u[i];
  *(u32x4*)(out + row * o_st + pc * 16) = pack8<T>(o);
}

// ------------------------------------------------------------------ q/k norm + rope + stores
struct QkArgs {
  const char* qkv;      // (N, (Hq + 2 Hkv) * D)
  char* q_out;          // (N, Hq, D) contiguous
  char* k_out;          // (N, Hkv, D) contiguous or null
  char* k_cache;        // flat (num_slots, Hkv * D)
  char* v_cache;
  char* q_cache;        // (max_seqs, window, Hq, D) or null
  const char* qn_w;     // (D,)
  const char* kn_w;
  const float* cos;     // (max_position, D/2)
  const float* sin;
  const int32_t* positions;     // (N,)
  const int32_t* slot_mapping;  // (N,) or null
  const int32_t* ring;          // (N, 3) triples aligned with the tokens, or null
  int N, Hq, Hkv, D, max_position, max_seqs, window;
  int64_t qkv_st, num_slots, qc_sseq, qc_sslot;
  float eps;
};

// One wave per head vector: lane i holds elements i and i + D/2, the two halves the NeoX
// rotation mixes, so norm, rotation and all stores need no exchange beyond one wave reduction.
template <typename T>
__global__ __launch_bounds__(kThreads) void qk_norm_rope_kernel(QkArgs a) {
  const int n = blockIdx.x, lane = threadIdx.x & 63;
  const int wv = blockIdx.y * kWaves + (threadIdx.x >> 6);
  const int nwv = gridDim.y * kWaves;
  const int half = a.D / 2;
  const bool on = lane < half;
  const int total = a.Hq + 2 * a.Hkv;
  int pos = a.positions[n];
  pos = min(max(pos, 0), a.max_position - 1);
  const float c = on ? a.cos[(int64_t)pos * half + lane] : 0.f;
  const float s = on ? a.sin[(int64_t)pos * half + lane] : 0.f;
  int64_t slot = a.slot_mapping ? a.slot_mapping[n] : -1;
  if (slot >= a.num_slots) slot = -1;
  int ring_seq = -1, ring_slot = -1;
  if (a.ring && a.q_cache && a.ring[n * 3] == n) {
    ring_seq = a.ring[n * 3 + 1];
    ring_slot = a.ring[n * 3 + 2];
    if (ring_seq < 0 || ring_seq >= a.max_seqs || ring_slot < 0 || ring_slot >= a.window) ring_seq = -1;
  }
  const uint16_t* src_row = (const uint16_t*)(a.qkv + (int64_t)n * a.qkv_st * 2);
  for (int hv = wv; hv < total; hv += nwv) {
    const uint16_t* src = src_row + (int64_t)hv * a.D;
    if (hv >= a.Hq + a.Hkv) {          // V: plain copy into the cache
      if (slot >= 0 && on) {
        uint16_t* dst = (uint16_t*)a.v_cache + (slot * a.Hkv + (hv - a.Hq - a.Hkv)) * a.D;
        dst[lane] = src[lane];
        dst[lane + half] = src[lane + half];
      }
      continue;
    }
    const bool is_q = hv < a.Hq;
    float x1 = on ? Elem<T>::ld(src, lane) : 0.f;
    float x2 = on ? Elem<T>::ld(src, lane + half) : 0.f;
    const float ss = wave_sum(x1 * x1 + x2 * x2);
    const float rs = rsqrtf(ss / (float)a.D + a.eps);
    const void* w = is_q ? a.qn_w : a.kn_w;
    if (on) {
      x1 = Elem<T>::rnd(Elem<T>::rnd(x1 * rs) * Elem<T>::ld(w, lane));
      x2 = Elem<T>::rnd(Elem<T>::rnd(x2 * rs) * Elem<T>::ld(w, lane + half));
      const uint16_t y1 = to_bits<T>(x1 * c - x2 * s);
      const uint16_t y2 = to_bits<T>(x2 * c + x1 * s);
      if (is_q) {
        uint16_t* dst = (uint16_t*)a.q_out + ((int64_t)n * a.Hq + hv) * a.D;
        dst[lane] = y1;
        dst[lane + half] = y2;
        if (ring_seq >= 0) {
          uint16_t* rq = (uint16_t*)a.q_cache + ring_seq * a.qc_sseq + ring_slot * a.qc_sslot +
                         (int64_t)hv * a.D;
          rq[lane] = y1;
          rq[lane + half] = y2;
        }
      } else {
        if (slot >= 0) {
          uint16_t* dst = (uint16_t*)a.k_cache + (slot * a.Hkv + (hv - a.Hq)) * a.D;
          dst[lane] = y1;
          dst[lane + half] = y2;
        }
        if (a.k_out) {
          uint16_t* dst = (uint16_t*)a.k_out + ((int64_t)n * a.Hkv + (hv - a.Hq)) * a.D;
          dst[lane] = y1;
          dst[lane + half] = y2;
        }
      }
    }
  }
}

}  // namespace

#define ZP_16BIT_ONLY(name)                                           \
  if (dtype != ZP_BF16 && dtype != ZP_F16) {                          \
    zp_set_error(name ": only 16-bit activations are supported");     \
    return ZP_EUNSUPPORTED;                                           \
  }

extern "C" int zp_add_rms_norm(const void* x, void* residual, const void* weight, void* out,
                               int32_t n, int32_t hidden, int64_t x_stride, int64_t r_stride,
                               int64_t out_stride, float eps, int32_t dtype, void* stream) {
  ZP_REQUIRE(n >= 0 && hidden > 0, "add_rms_norm: bad dims");
  ZP_16BIT_ONLY("add_rms_norm");
  if (hidden % 8 != 0 || hidden > 8 * kThreads * kMaxPieces) {
    zp_set_error("add_rms_norm: hidden %d unsupported (multiple of 8, <= %d)", hidden,
                 8 * kThreads * kMaxPieces);
    return ZP_EUNSUPPORTED;
  }
  if (n == 0) return ZP_OK;
  ZP_REQUIRE(x && weight && out, "add_rms_norm: null pointer");
  ZP_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)weight % 16 == 0 &&
                 (uintptr_t)residual % 16 == 0 && x_stride % 8 == 0 && out_stride % 8 == 0 &&
                 r_stride % 8 == 0,
             "add_rms_norm: rows must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
#define ZP_ARN(T, ADD)                                                                          \
  hipLaunchKernelGGL((add_rms_kernel<T, ADD>), dim3(n), dim3(kThreads), 0, st, (const char*)x,  \
                     (char*)residual, (const char*)weight, (char*)out, hidden, x_stride * 2,    \
                     r_stride * 2, out_stride * 2, eps)
  if (dtype == ZP_BF16) { if (residual) ZP_ARN(BF16, true); else ZP_ARN(BF16, false); }
  else                  { if (residual) ZP_ARN(F16, true);  else ZP_ARN(F16, false); }
#undef ZP_ARN
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

extern "C" int zp_silu_and_mul(const void* gate_up, void* out, int32_t n, int32_t intermediate,
                               int64_t gu_stride, int64_t out_stride, int32_t dtype, void* stream) {
  ZP_REQUIRE(n >= 0 && intermediate > 0, "silu_and_mul: bad dims");
  ZP_16BIT_ONLY("silu_and_mul");
  if (intermediate % 8 != 0) {
    zp_set_error("silu_and_mul: intermediate size %d is not a multiple of 8", intermediate);
    return ZP_EUNSUPPORTED;
  }
  if (n == 0) return ZP_OK;
  ZP_REQUIRE(gate_up && out, "silu_and_mul: null pointer");
  ZP_REQUIRE((uintptr_t)gate_up % 16 == 0 && (uintptr_t)out % 16 == 0 && gu_stride % 8 == 0 &&
                 out_stride % 8 == 0,
             "silu_and_mul: rows must be 16-byte aligned");
  const int ppr = intermediate / 8;
  const int64_t total = (int64_t)n * ppr;
  const unsigned grid = (unsigned)((total + kThreads - 1) / kThreads);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == ZP_BF16)
    hipLaunchKernelGGL((silu_mul_kernel<BF16>), dim3(grid), dim3(kThreads), 0, st,
                       (const char*)gate_up, (char*)out, ppr, total, gu_stride * 2, out_stride * 2,
                       (int64_t)intermediate * 2);
  else
    hipLaunchKernelGGL((silu_mul_kernel<F16>), dim3(grid), dim3(kThreads), 0, st,
                       (const char*)gate_up, (char*)out, ppr, total, gu_stride * 2, out_stride * 2,
                       (int64_t)intermediate * 2);
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

extern "C" int zp_qk_norm_rope_store(const void* qkv, void* q_out, void* k_out, void* k_cache,
                                     void* v_cache,
                                     void* query_cache, const void* q_norm_weight,
                                     const void* k_norm_weight, const float* cos, const float* sin,
                                     const int32_t* positions, const int32_t* slot_mapping,
                                     const int32_t* query_triples, int32_t n, int32_t Hq,
                                     int32_t Hkv, int32_t D, int32_t max_position,
                                     int64_t qkv_stride, int64_t num_slots, int32_t max_seqs,
                                     int32_t window, int64_t qc_stride_seq, int64_t qc_stride_slot,
                                     float eps, int32_t dtype, void* stream) {
  ZP_REQUIRE(n >= 0 && Hq > 0 && Hkv > 0 && D > 0 && max_position > 0, "qk_norm_rope_store: bad dims");
  ZP_16BIT_ONLY("qk_norm_rope_store");
  if (D % 2 != 0 || D > 128) {
    zp_set_error("qk_norm_rope_store: head_dim %d unsupported (even, <= 128)", D);
    return ZP_EUNSUPPORTED;
  }
  if (n == 0) return ZP_OK;
  ZP_REQUIRE(qkv && q_out && q_norm_weight && k_norm_weight && cos && sin && positions,
             "qk_norm_rope_store: null pointer");
  ZP_REQUIRE(!slot_mapping || (k_cache && v_cache), "qk_norm_rope_store: slot mapping without caches");
  QkArgs a;
  a.qkv = (const char*)qkv; a.q_out = (char*)q_out; a.k_out = (char*)k_out; a.k_cache = (char*)k_cache;
  a.v_cache = (char*)v_cache; a.q_cache = (char*)query_cache; a.qn_w = (const char*)q_norm_weight;
  a.kn_w = (const char*)k_norm_weight; a.cos = cos; a.sin = sin; a.positions = positions;
  a.slot_mapping = slot_mapping; a.ring = query_triples; a.N = n; a.Hq = Hq; a.Hkv = Hkv; a.D = D;
  a.max_position = max_position; a.max_seqs = max_seqs; a.window = window; a.qkv_st = qkv_stride;
  a.num_slots = num_slots; a.qc_sseq = qc_stride_seq; a.qc_sslot = qc_stride_slot; a.eps = eps;
  hipStream_t st = (hipStream_t)stream;
  const int total = Hq + 2 * Hkv;
  const unsigned gy = (unsigned)((total + 3 * kWaves - 1) / (3 * kWaves));   // ~3 vectors per wave
  if (dtype == ZP_BF16)
    hipLaunchKernelGGL((qk_norm_rope_kernel<BF16>), dim3(n, gy), dim3(kThreads), 0, st, a);
  else
    hipLaunchKernelGGL((qk_norm_rope_kernel<F16>), dim3(n, gy), dim3(kThreads), 0, st, a);
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}
