// Bandwidth-bound elementwise / row-wise stages between the scorer and the selector:
// global-score carry-over, sequence-axis pooling, the fused score epilogue
// (max-normalise, redundancy combine, attention sink, window mask, pad mask) and the
// key L2 norm.  Rounding follows the reference's torch/Triton ops: every op that the
// reference runs on a cache-dtype tensor rounds its result to that dtype.
#include "common.h"
#include <math.h>

namespace {

constexpr int kThreads = 256;

// ------------------------------------------------------------------ global score
// One workgroup per (layer, sequence, page); threads walk the page of the score cache
// in its own (slot-major, head-minor) order so cache accesses are fully coalesced.
template <typename T>
__global__ __launch_bounds__(kThreads) void global_score_kernel(
    void* __restrict__ scores, void* __restrict__ cache, const int32_t* __restrict__ table,
    const uint8_t* __restrict__ compressed, int B, int NB, int BS, int Hkv, int num_pages,
    int64_t c_sl, int64_t c_sp, float decay, int method, int write_cache) {
  const int j = blockIdx.x % NB;
  const int b = (blockIdx.x / NB) % B;
  const int l = blockIdx.x / (NB * B);
  const int code = table[(int64_t)b * NB + j];
  if (page_is_pad(code)) return;
  const int pid = page_id(code);
  if (pid >= num_pages) return;
  const bool carry = compressed[b] != 0 && !page_is_last(code);
  if (!carry && !write_cache) return;   // nothing to add and nothing to write back
  const int64_t sbase = (((int64_t)l * B + b) * Hkv) * (int64_t)NB * BS + (int64_t)j * BS;
  const int64_t cbase = l * c_sl + pid * c_sp;
  const int n = BS * Hkv;
  for (int c = threadIdx.x; c < n; c += kThreads) {
    const int slot = c / Hkv, h = c - slot * Hkv;
    const int64_t si = sbase + (int64_t)h * NB * BS + slot;
    float v = Elem<T>::ld(scores, si);
    if (carry) {
      const float old = Elem<T>::ld(cache, cbase + c) * decay;
      v = Elem<T>::rnd(method == ZP_ACTIVATE_MAX ? fmaxf(v, old) : v + old);
      Elem<T>::st(scores, si, v);
    }
    if (write_cache) Elem<T>::st(cache, cbase + c, v);
  }
}

// ------------------------------------------------------------------ pooling
template <typename T>
__global__ __launch_bounds__(kThreads) void pool_kernel(
    const void* __restrict__ in, void* __restrict__ out, const uint8_t* __restrict__ compressed,
    int B, int Hkv, int Tn, int ksize, int continues, int mode) {
  extern __shared__ float row[];
  const uint32_t r = blockIdx.x;          // 32-bit: a 64-bit division costs hundreds of scalar instructions
  const int b = (int)((r / (uint32_t)Hkv) % (uint32_t)B);
  const int64_t base = (int64_t)r * Tn;
  const bool raw = !continues && compressed[b] != 0;
  if (raw) {
    for (int t = threadIdx.x; t < Tn; t += kThreads)
      Elem<T>::st(out, base + t, Elem<T>::ld(in, base + t));
    return;
  }
  for (int t = threadIdx.x; t < Tn; t += kThreads) row[t] = Elem<T>::ld(in, base + t);
  __syncthreads();
  const int half = ksize / 2;
  for (int t = threadIdx.x; t < Tn; t += kThreads) {
    const int lo = max(t - half, 0), hi = min(t + half, Tn - 1);
    float acc;
    if (mode == ZP_POOL_MAX) {
      acc = row[lo];
      for (int i = lo + 1; i <= hi; ++i) acc = fmaxf(acc, row[i]);
    } else {
      acc = 0.f;
      for (int i = lo; i <= hi; ++i) acc += row[i];
      acc = acc / (float)ksize;
    }
    Elem<T>::st(out, base + t, acc);
  }
}

// ------------------------------------------------------------------ score epilogue
__device__ __forceinline__ float block_max(float v, float* lds) {
  v = wave_max(v);
  __syncthreads();
  if (lane_id() == 0) lds[wave_id()] = v;
  __syncthreads();
  float m = lds[0];
#pragma unroll
  for (int i = 1; i < kThreads / 64; ++i) m = fmaxf(m, lds[i]);
  return m;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void epilogue_kernel(
    void* __restrict__ scores, const void* __restrict__ red, const int32_t* __restrict__ table,
    int B, int NB, int BS, int Hkv, int norm_s, int norm_r, float lam, float one_minus_lam,
    int sink_len, int window, int mask_pad) {
  __shared__ float red_lds[kThreads / 64];
  const uint32_t r = blockIdx.x;          // 32-bit: a 64-bit division costs hundreds of scalar instructions
  const int b = (int)((r / (uint32_t)Hkv) % (uint32_t)B);
  const int Tn = NB * BS;
  const int64_t base = (int64_t)r * Tn;
  const int32_t* trow = table + (int64_t)b * NB;
  float smax = 1.f, rmax = 1.f;
  if (norm_s) {
    float m = -INFINITY;
    for (int t = threadIdx.x; t < Tn; t += kThreads) m = fmaxf(m, Elem<T>::ld(scores, base + t));
    smax = block_max(m, red_lds);
  }
  if (norm_r && red) {
    float m = -INFINITY;
    for (int t = threadIdx.x; t < Tn; t += kThreads) m = fmaxf(m, Elem<T>::ld(red, base + t));
    rmax = block_max(m, red_lds);
  }
  for (int t = threadIdx.x; t < Tn; t += kThreads) {
    const int j = t / BS, slot = t - j * BS;
    const int code = trow[j];
    float v = Elem<T>::ld(scores, base + t);
    if (norm_s) v = Elem<T>::rnd(v / smax);
    if (red) {
      float rv = Elem<T>::ld(red, base + t);
      if (norm_r) rv = Elem<T>::rnd(rv / rmax);
      const float a = Elem<T>::rnd(v * lam);
      const float c = Elem<T>::rnd(rv * one_minus_lam);
      v = Elem<T>::rnd(a - c);
    }
    if (t < sink_len) v = INFINITY;
    if (window > 0 && page_is_last(code) && slot >= BS - window) v = INFINITY;
    if (mask_pad && page_is_pad(code)) v = -INFINITY;
    Elem<T>::st(scores, base + t, v);
  }
}

// ------------------------------------------------------------------ key norm
// One workgroup per (layer, sequence, page).  A group of LPV lanes owns one key vector
// (16 bytes per lane), reduces its squares with xor-shuffles.
template <typename T>
__device__ __forceinline__ float sumsq16(const vec16& v);
template <> __device__ __forceinline__ float sumsq16<F32>(const vec16& v) {
  float a = __uint_as_float(v.x), b = __uint_as_float(v.y), c = __uint_as_float(v.z),
        d = __uint_as_float(v.w);
  return a * a + b * b + c * c + d * d;
}
template <> __device__ __forceinline__ float sumsq16<BF16>(const vec16& v) {
  float s = 0.f;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float lo = __uint_as_float(w[i] << 16), hi = __uint_as_float(w[i] & 0xffff0000u);
    s += lo * lo;
    s += hi * hi;
  }
  return s;
}
template <> __device__ __forceinline__ float sumsq16<F16>(const vec16& v) {
  float s = 0.f;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float lo = f16_bits_to_float((uint16_t)(w[i] & 0xffffu)), hi = f16_bits_to_float((uint16_t)(w[i] >> 16));
    s += lo * lo;
    s += hi * hi;
  }
  return s;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void key_norm_kernel(
    const char* __restrict__ k, const int32_t* __restrict__ table, void* __restrict__ out, int B,
    int NB, int BS, int Hkv, int D, int num_pages, int64_t k_sl, int64_t k_sp, float eps,
    int lpv /* 0: generic path */) {
  const int j = blockIdx.x % NB;
  const int b = (blockIdx.x / NB) % B;
  const int l = blockIdx.x / (NB * B);
  const int code = table[(int64_t)b * NB + j];
  const int64_t obase = (((int64_t)l * B + b) * Hkv) * (int64_t)NB * BS + (int64_t)j * BS;
  const int nvec = BS * Hkv;
  const float epsr = Elem<T>::rnd(eps);
  const int pid = page_is_pad(code) ? -1 : page_id(code);
  if (pid < 0 || pid >= num_pages) {  // pad page: norm 0 clamped to eps
    for (int c = threadIdx.x; c < nvec; c += kThreads) {
      const int slot = c / Hkv, h = c - slot * Hkv;
      Elem<T>::st(out, obase + (int64_t)h * NB * BS + slot, epsr);
    }
    return;
  }
  const char* page = k + (l * k_sl + pid * k_sp) * T::bytes;
  if (lpv > 0) {
    const int vec_per_iter = kThreads / lpv;
    const int sub = threadIdx.x % lpv, vi = threadIdx.x / lpv;
    for (int c0 = 0; c0 < nvec; c0 += vec_per_iter) {
      const int c = c0 + vi;
      float s = 0.f;
      if (c < nvec) {
        const vec16 v = *(const vec16*)(page + ((int64_t)c * D) * T::bytes + sub * 16);
        s = sumsq16<T>(v);
      }
      for (int o = lpv >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
      if (c < nvec && sub == 0) {
        const int slot = c / Hkv, h = c - slot * Hkv;
        const float nv = fmaxf(Elem<T>::rnd(sqrtf(s)), epsr);
        Elem<T>::st(out, obase + (int64_t)h * NB * BS + slot, nv);
      }
    }
  } else {
    for (int c = threadIdx.x; c < nvec; c += kThreads) {
      float s = 0.f;
      for (int d = 0; d < D; ++d) {
        const float x = Elem<T>::ld(page, (int64_t)c * D + d);
        s += x * x;
      }
      const int slot = c / Hkv, h = c - slot * Hkv;
      const float nv = fmaxf(Elem<T>::rnd(sqrtf(s)), epsr);
      Elem<T>::st(out, obase + (int64_t)h * NB * BS + slot, nv);
    }
  }
}

}  // namespace

extern "C" int zp_global_score(void* scores, void* score_cache, const int32_t* block_table,
                               const uint8_t* compressed, int32_t L, int32_t B, int32_t NB,
                               int32_t BS, int32_t Hkv, int32_t num_pages, int64_t c_sl,
                               int64_t c_sp, float decay_factor, int32_t activate_method,
                               int32_t write_cache, int32_t dtype, void* stream) {
  ZP_REQUIRE(scores && score_cache && block_table && compressed, "global_score: null pointer");
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0, "global_score: bad dims");
  ZP_REQUIRE(decay_factor >= 0.f && decay_factor <= 1.f, "global_score: decay_factor %g outside [0,1]",
             (double)decay_factor);
  ZP_REQUIRE(activate_method == ZP_ACTIVATE_MAX || activate_method == ZP_ACTIVATE_SUM,
             "global_score: unknown activate_method %d", activate_method);
  if (L == 0 || B == 0) return ZP_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)((int64_t)L * B * NB));
  ZP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((global_score_kernel<T>), grid, dim3(kThreads), 0, st,
                                              scores, score_cache, block_table, compressed, B, NB,
                                              BS, Hkv, num_pages, c_sl, c_sp, decay_factor,
                                              activate_method, write_cache));
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

extern "C" int zp_pool_scores(const void* scores_in, void* scores_out, const uint8_t* compressed,
                              int32_t L, int32_t B, int32_t Hkv, int32_t Tn, int32_t kernel_size,
                              int32_t continues_pooling, int32_t mode, int32_t dtype,
                              void* stream) {
  ZP_REQUIRE(scores_in && scores_out && compressed, "pool_scores: null pointer");
  ZP_REQUIRE(scores_in != scores_out, "pool_scores: in and out must be distinct buffers");
  ZP_REQUIRE(L >= 0 && B >= 0 && Hkv > 0 && Tn > 0, "pool_scores: bad dims");
  ZP_REQUIRE(kernel_size >= 1 && (kernel_size & 1), "pool_scores: kernel_size %d must be odd",
             kernel_size);
  ZP_REQUIRE(mode == ZP_POOL_MAX || mode == ZP_POOL_AVG, "pool_scores: unknown mode %d", mode);
  ZP_REQUIRE((int64_t)Tn * 4 <= 160 * 1024 - 1024, "pool_scores: row of %d tokens exceeds LDS", Tn);
  if (L == 0 || B == 0) return ZP_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)((int64_t)L * B * Hkv));
  const size_t smem = (size_t)Tn * 4;
#define ZP_POOL_LAUNCH()                                                                          \
  do {                                                                                            \
    if (smem > 64 * 1024 &&                                                                       \
        hipFuncSetAttribute((const void*)pool_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                            (int)smem) != hipSuccess) {                                           \
      zp_set_error("pool_scores: cannot reserve %zu bytes of LDS", smem);                         \
      return ZP_EHIP;                                                                             \
    }                                                                                             \
    hipLaunchKernelGGL((pool_kernel<T>), grid, dim3(kThreads), smem, st, scores_in, scores_out,   \
                       compressed, B, Hkv, Tn, kernel_size, continues_pooling, mode);             \
  } while (0)
  ZP_DISPATCH_DTYPE(dtype, ZP_POOL_LAUNCH());
#undef ZP_POOL_LAUNCH
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

extern "C" int zp_score_epilogue(void* scores, const void* redundancy, const int32_t* block_table,
                                 int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                                 int32_t max_norm_scores, int32_t max_norm_red,
                                 double redudancy_lambda, int32_t sink_len, int32_t window,
                                 int32_t mask_pad, int32_t dtype, void* stream) {
  ZP_REQUIRE(scores && block_table, "score_epilogue: null pointer");
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0, "score_epilogue: bad dims");
  ZP_REQUIRE(window >= 0 && window <= BS, "score_epilogue: window %d outside [0, BS=%d]", window, BS);
  ZP_REQUIRE(sink_len >= 0, "score_epilogue: negative sink_len");
  if (L == 0 || B == 0) return ZP_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)((int64_t)L * B * Hkv));
  const float lam = (float)redudancy_lambda, oml = (float)(1.0 - redudancy_lambda);
  ZP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((epilogue_kernel<T>), grid, dim3(kThreads), 0, st, scores,
                                              redundancy, block_table, B, NB, BS, Hkv,
                                              max_norm_scores, max_norm_red, lam, oml, sink_len,
                                              window, mask_pad));
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

extern "C" int zp_key_norm(const void* k_cache, const int32_t* block_table, void* norm_out,
                           int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv, int32_t D,
                           int32_t num_pages, int64_t k_sl, int64_t k_sp, float norm_epsilon,
                           int32_t dtype, void* stream) {
  ZP_REQUIRE(k_cache && block_table && norm_out, "key_norm: null pointer");
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0 && D > 0, "key_norm: bad dims");
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "key_norm: unknown dtype tag %d", dtype);
  if (L == 0 || B == 0) return ZP_OK;
  const int es = zp_dtype_bytes(dtype);
  const int64_t vec = (int64_t)D * es;
  int lpv = 0;
  if (vec % 16 == 0 && ((uintptr_t)k_cache % 16) == 0 && (k_sl * es) % 16 == 0 &&
      (k_sp * es) % 16 == 0) {
    const int64_t n = vec / 16;
    if (n <= 64 && (n & (n - 1)) == 0) lpv = (int)n;
  }
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)((int64_t)L * B * NB));
  ZP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((key_norm_kernel<T>), grid, dim3(kThreads), 0, st,
                                              (const char*)k_cache, block_table, norm_out, B, NB,
                                              BS, Hkv, D, num_pages, k_sl, k_sp, norm_epsilon, lpv));
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}
