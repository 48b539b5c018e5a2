// The two cache-side kernels of the decode step that surround the compression path:
// scattering the new token's K/V into the paged cache, and single-query attention over a
// sequence's pages.  Both are HBM-streaming kernels (the decode step reads every cached K and V
// once): 16 lanes own one 256-byte head vector, four token rows per wave instruction.
#include "common.h"
#include <math.h>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------ store_kvcache
template <typename P>
__global__ __launch_bounds__(kThreads) void store_kv_kernel(
    const char* __restrict__ key, const char* __restrict__ value, char* __restrict__ kc,
    char* __restrict__ vc, const int32_t* __restrict__ slot_mapping, int pieces, int64_t k_st,
    int64_t v_st, int64_t row_bytes, int64_t num_slots) {
  const int idx = blockIdx.x;
  const int64_t slot = slot_mapping[idx];
  if (slot < 0 || slot >= num_slots) return;
  const P* ks = (const P*)(key + idx * k_st);
  const P* vs = (const P*)(value + idx * v_st);
  P* kd = (P*)(kc + slot * row_bytes);
  P* vd = (P*)(vc + slot * row_bytes);
  for (int i = threadIdx.x; i < pieces; i += kThreads) {
    kd[i] = ks[i];
    vd[i] = vs[i];
  }
}

// ------------------------------------------------------------------ paged decode attention
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

struct DecodeArgs {
  const char* q;       // (B, Hq, D)
  const char* k;       // (pages, BS, Hkv, D) one layer
  const char* v;
  const int32_t* table;  // (B, NB) plain page ids, -1 pad
  const int32_t* ctx;    // (B,) tokens to attend to
  void* out;           // (B, Hq, D)
  int B, Hq, Hkv, G, D, BS, NB, num_pages;
  int64_t k_sp, v_sp;  // page strides in elements
  float scale;
};

// One workgroup per (sequence, kv head); G <= 8 query heads share the K/V stream.
// Pass 1 writes scaled logits (G x T) to LDS, pass 2 the softmax statistics, pass 3 P.V.
template <typename T, int G>
__global__ __launch_bounds__(kThreads) void paged_decode_kernel(DecodeArgs p) {
  extern __shared__ __align__(16) float lds[];
  __shared__ float red[kWaves * G];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = tid >> 4, sub = tid & 15;     // 16 groups of 16 lanes
  const int h = blockIdx.x % p.Hkv, b = blockIdx.x / p.Hkv;
  int Tn = p.ctx[b];
  Tn = max(0, min(Tn, p.NB * p.BS));
  const int Tpad = (p.NB * p.BS + 15) & ~15;
  float* logit = lds;                            // [G][Tpad]
  const int dvalid = p.D / 8;                    // 16-byte pieces per head vector (<= 16)
  const bool on = sub < dvalid;
  const int64_t row = (int64_t)p.Hkv * p.D * 2;
  const int64_t hoff = (int64_t)h * p.D * 2 + sub * 16;

  // query pieces of the G heads
  float qf[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (on) raw = *(const u32x4*)(p.q + (((int64_t)b * p.Hq + h * G + g) * p.D) * 2 + sub * 16);
    unpack8<T>(raw, qf[g]);
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[g][i] *= p.scale;
  }
  const int32_t* trow = p.table + (int64_t)b * p.NB;

  // ---- pass 1: logits
  for (int t0 = 0; t0 < Tn; t0 += 16 * 4) {
    u32x4 raw[4];
    int tt[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = t0 + u * 16 + grp;
      tt[u] = t;
      const int tc = min(t, Tn - 1);
      int pid = trow[tc / p.BS];
      pid = (pid >= 0 && pid < p.num_pages) ? pid : 0;
      raw[u] = *(const u32x4*)(p.k + (int64_t)pid * p.k_sp * 2 + (int64_t)(tc % p.BS) * row +
                               (on ? hoff : (int64_t)h * p.D * 2));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float kf[8];
      unpack8<T>(raw[u], kf);
      float s[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float a = 0.f;
        if (on) {
#pragma unroll
          for (int i = 0; i < 8; ++i) a += qf[g][i] * kf[i];
        }
        s[g] = a;
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) {
#pragma unroll
        for (int g = 0; g < G; ++g) s[g] += __shfl_xor(s[g], o, 64);
      }
      if (sub == 0 && tt[u] < Tn) {
#pragma unroll
        for (int g = 0; g < G; ++g) logit[g * Tpad + tt[u]] = s[g];
      }
    }
  }
  __syncthreads();
  // ---- pass 2: softmax statistics per head
  float mx[G], inv[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float m = -INFINITY;
    for (int t = tid; t < Tn; t += kThreads) m = fmaxf(m, logit[g * Tpad + t]);
    m = wave_max(m);
    if (lane == 0) red[wave * G + g] = m;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float m = red[g];
    for (int w = 1; w < kWaves; ++w) m = fmaxf(m, red[w * G + g]);
    mx[g] = m;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float s = 0.f;
    for (int t = tid; t < Tn; t += kThreads) {
      const float e = __expf(logit[g * Tpad + t] - mx[g]);
      logit[g * Tpad + t] = e;
      s += e;
    }
    s = wave_sum(s);
    if (lane == 0) red[wave * G + g] = s;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float s = 0.f;
    for (int w = 0; w < kWaves; ++w) s += red[w * G + g];
    inv[g] = s > 0.f ? 1.f / s : 0.f;
  }
  // ---- pass 3: P.V, each 16-lane group accumulates its tokens
  float acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
  for (int t0 = 0; t0 < Tn; t0 += 16 * 4) {
    u32x4 raw[4];
    int tt[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = t0 + u * 16 + grp;
      tt[u] = t;
      const int tc = min(t, Tn - 1);
      int pid = trow[tc / p.BS];
      pid = (pid >= 0 && pid < p.num_pages) ? pid : 0;
      raw[u] = *(const u32x4*)(p.v + (int64_t)pid * p.v_sp * 2 + (int64_t)(tc % p.BS) * row +
                               (on ? hoff : (int64_t)h * p.D * 2));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float vf[8];
      unpack8<T>(raw[u], vf);
      if (tt[u] < Tn) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float pw = logit[g * Tpad + tt[u]];
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[g][i] += pw * vf[i];
        }
      }
    }
  }
  __syncthreads();  // logits no longer needed: reuse the LDS for the cross-group reduction
  float* part = lds;  // [16 groups][G][128]
  if (on) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < 8; ++i) part[(grp * G + g) * 128 + sub * 8 + i] = acc[g][i];
  }
  __syncthreads();
  for (int e = tid; e < G * p.D; e += kThreads) {
    const int g = e / p.D, d = e - g * p.D;
    float s = 0.f;
#pragma unroll
    for (int q = 0; q < 16; ++q) s += part[(q * G + g) * 128 + d];
    Elem<T>::st(p.out, ((int64_t)b * p.Hq + h * G + g) * p.D + d, s * inv[g]);
  }
}

template <typename T, int G>
int launch_decode(const DecodeArgs& a, hipStream_t st) {
  const int Tpad = (a.NB * a.BS + 15) & ~15;
  size_t smem = sizeof(float) * (size_t)G * Tpad;
  const size_t part = sizeof(float) * 16 * G * 128;
  if (part > smem) smem = part;
  if (smem > 150 * 1024) {
    zp_set_error("paged_decode_attention: %d cached tokens x %d heads exceed LDS", a.NB * a.BS, G);
    return ZP_EUNSUPPORTED;
  }
  if (smem > 64 * 1024 &&
      hipFuncSetAttribute((const void*)paged_decode_kernel<T, G>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    zp_set_error("paged_decode_attention: cannot reserve %zu bytes of LDS", smem);
    return ZP_EHIP;
  }
  hipLaunchKernelGGL((paged_decode_kernel<T, G>), dim3((unsigned)(a.B * a.Hkv)), dim3(kThreads), smem,
                     st, a);
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

template <typename T>
int dispatch_group(const DecodeArgs& a, hipStream_t st) {
  switch (a.G) {
    case 1: return launch_decode<T, 1>(a, st);
    case 2: return launch_decode<T, 2>(a, st);
    case 4: return launch_decode<T, 4>(a, st);
    case 8: return launch_decode<T, 8>(a, st);
    default:
      zp_set_error("paged_decode_attention: GQA group %d unsupported (1, 2, 4, 8)", a.G);
      return ZP_EUNSUPPORTED;
  }
}

}  // namespace

extern "C" int zp_store_kvcache(const void* key, const void* value, void* k_cache, void* v_cache,
                                const int32_t* slot_mapping, int32_t n, int32_t row_elems,
                                int64_t key_stride, int64_t value_stride, int64_t num_slots,
                                int32_t dtype, void* stream) {
  ZP_REQUIRE(n >= 0 && row_elems > 0, "store_kvcache: bad dims");
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "store_kvcache: unknown dtype tag %d", dtype);
  if (n == 0) return ZP_OK;
  ZP_REQUIRE(key && value && k_cache && v_cache && slot_mapping, "store_kvcache: null pointer");
  const int es = zp_dtype_bytes(dtype);
  const int64_t rb = (int64_t)row_elems * es;
  int piece = 2;
  for (int cand : {16, 8, 4}) {
    if (rb % cand == 0 && (key_stride * es) % cand == 0 && (value_stride * es) % cand == 0 &&
        (uintptr_t)key % cand == 0 && (uintptr_t)value % cand == 0 &&
        (uintptr_t)k_cache % cand == 0 && (uintptr_t)v_cache % cand == 0) {
      piece = cand;
      break;
    }
  }
  hipStream_t st = (hipStream_t)stream;
  const int pieces = (int)(rb / piece);
#define ZP_SKV(P)                                                                              \
  hipLaunchKernelGGL((store_kv_kernel<P>), dim3(n), dim3(kThreads), 0, st, (const char*)key,   \
                     (const char*)value, (char*)k_cache, (char*)v_cache, slot_mapping, pieces, \
                     key_stride * es, value_stride * es, rb, num_slots)
  switch (piece) {
    case 16: ZP_SKV(u32x4); break;
    case 8:  ZP_SKV(uint2); break;
    case 4:  ZP_SKV(uint32_t); break;
    default: ZP_SKV(uint16_t); break;
  }
#undef ZP_SKV
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

extern "C" int zp_paged_decode_attention(const void* q, const void* k_cache, const void* v_cache,
                                         const int32_t* block_tables, const int32_t* context_lens,
                                         void* out, int32_t B, int32_t Hq, int32_t Hkv, int32_t D,
                                         int32_t BS, int32_t NB, int32_t num_pages,
                                         int64_t k_stride_page, int64_t v_stride_page,
                                         float softmax_scale, int32_t dtype, void* stream) {
  ZP_REQUIRE(q && k_cache && v_cache && block_tables && context_lens && out,
             "paged_decode_attention: null pointer");
  ZP_REQUIRE(B >= 0 && Hq > 0 && Hkv > 0 && D > 0 && BS > 0 && NB > 0,
             "paged_decode_attention: bad dims");
  ZP_REQUIRE(Hq % Hkv == 0, "paged_decode_attention: Hq=%d not a multiple of Hkv=%d", Hq, Hkv);
  if (dtype != ZP_BF16 && dtype != ZP_F16) {
    zp_set_error("paged_decode_attention: only 16-bit caches are supported");
    return ZP_EUNSUPPORTED;
  }
  if (D % 8 != 0 || D > 128) {
    zp_set_error("paged_decode_attention: head_dim %d unsupported (multiple of 8, <= 128)", D);
    return ZP_EUNSUPPORTED;
  }
  ZP_REQUIRE((uintptr_t)q % 16 == 0 && (uintptr_t)k_cache % 16 == 0 && (uintptr_t)v_cache % 16 == 0 &&
                 (k_stride_page * 2) % 16 == 0 && (v_stride_page * 2) % 16 == 0,
             "paged_decode_attention: tensors must be 16-byte aligned");
  if (B == 0) return ZP_OK;
  DecodeArgs a;
  a.q = (const char*)q; a.k = (const char*)k_cache; a.v = (const char*)v_cache;
  a.table = block_tables; a.ctx = context_lens; a.out = out;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.G = Hq / Hkv; a.D = D; a.BS = BS; a.NB = NB;
  a.num_pages = num_pages; a.k_sp = k_stride_page; a.v_sp = v_stride_page; a.scale = softmax_scale;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == ZP_BF16) return dispatch_group<BF16>(a, st);
  return dispatch_group<F16>(a, st);
}
