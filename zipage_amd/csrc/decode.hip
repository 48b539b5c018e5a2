// The two cache-side kernels of the decode step that surround the compression path:
// scattering the new token's K/V into the paged cache, and single-query attention over a
// sequence's pages.  Both are HBM-streaming kernels: the decode step reads every cached K and V
// exactly once, so the attention kernel is organised around 16-byte loads that cover whole
// 128-byte lines of a (token, kv head) vector and around packed 16-bit dot products.
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
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// acc + a.lo*b.lo + a.hi*b.hi on packed 16-bit pairs, fp32 accumulate (v_dot2_f32_bf16 / _f16)
template <typename T> __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c);
template <> __device__ __forceinline__ float dot2<BF16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b),
                                         c, false);
}
template <> __device__ __forceinline__ float dot2<F16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<BF16>(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}
template <> __device__ __forceinline__ uint32_t pack2<F16>(float lo, float hi) {
  f16x2 v = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

// Sum over the 8 lanes of a row group, result in all 8 (three DPP stages, no LDS traffic).
__device__ __forceinline__ float group8_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  return v;
}

struct DecodeArgs {
  const char* q;       // (B, Hq, D)
  const char* k;       // (pages, BS, Hkv, D) one layer
  const char* v;
  const int32_t* table;  // (B, NB) plain page ids, -1 pad
  const int32_t* ctx;    // (B,) tokens to attend to
  void* out;           // (B, Hq, D)
  int B, Hq, Hkv, G, D, BS, NB, num_pages;
  int bs_shift;        // log2(BS) when BS is a power of two, else -1
  int chunk;           // tokens per slice when the context is walked in slices (multiple of 128)
  int64_t k_sp, v_sp;  // page strides in elements
  float scale;
};

// K and V rows are read exactly once per step: non-temporal loads stream them past L2
// (measured 5.7 -> 6.3 TB/s at 256 sequences x 2176 tokens).
#ifndef ZP_DEC_LOAD
#define ZP_DEC_LOAD(ptr) __builtin_nontemporal_load(ptr)
#endif
constexpr int kMaxTablePages = 256;     // block-table entries per sequence (the LDS logits cap the context first)
constexpr int kGroups = kThreads / 8;  // token rows in flight per step of the workgroup
constexpr int kUnroll = 4;             // rows per lane group and loop trip (must be even)

// One workgroup per (sequence, kv head); the G query heads of the group share the K/V stream.
// Eight lanes own one token row: lane `sub` holds the 16-byte pieces `sub` and `sub + 8` of the
// head vector, so one load instruction of the wave covers eight rows, each a full 128-byte line.
//   pass 1: logits = q.k on packed 16-bit pairs, reduced over the 8 lanes, scaled, to LDS (fp32)
//   pass 2: row maximum, p = exp(logit - max) summed in fp32; p is rounded to the cache dtype and
//           packed in pairs (token t, token t + 32) over the logit word of t
//   pass 3: out += p.v with two tokens per dot2 (the pair above), fp32 accumulate; the row
//           groups are summed at the end and scaled by 1 / sum(p).
template <typename T, int G, bool CHUNKED>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(G <= 4 && !CHUNKED ? 4 : 2, 4))) void paged_decode_kernel(DecodeArgs p) {
  extern __shared__ __align__(16) float lds[];
  __shared__ float red[kWaves * G];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = tid >> 3, sub = tid & 7;
  const int h = blockIdx.x % p.Hkv, b = blockIdx.x / p.Hkv;
  int Tn = p.ctx[b];
  Tn = max(0, min(Tn, p.NB * p.BS));
  const int Tpad = CHUNKED ? p.chunk : ((p.NB * p.BS + 63) & ~63);   // LDS row of one head's logits
  float* logit = lds;                            // [G][Tpad]
  uint32_t* pw = (uint32_t*)lds;                 // packed p pairs over the same words
  const int pieces = p.D / 8;                    // 16-byte pieces per head vector (<= 16)
  const bool onA = sub < pieces, onB = sub + 8 < pieces;
  const int64_t row = (int64_t)p.Hkv * p.D * 2;
  const int64_t offA = (int64_t)h * p.D * 2 + (onA ? sub * 16 : 0);
  const int64_t offB = (int64_t)h * p.D * 2 + (onB ? (sub + 8) * 16 : 0);
  // page ids of the sequence, validated once, in LDS: the row address needs no global lookup
  __shared__ int pages_lds[kMaxTablePages];
  for (int j = tid; j < p.NB; j += kThreads) {
    const int pid = p.table[(int64_t)b * p.NB + j];
    pages_lds[j] = (pid >= 0 && pid < p.num_pages) ? pid : 0;
  }
  __syncthreads();
  const u32x4 zero4 = {0u, 0u, 0u, 0u};

  auto row_base = [&](const char* cache, int64_t page_stride, int t) -> const char* {
    const int tc = min(t, Tn - 1);
    // page sizes are powers of two in practice: shifts instead of two integer divisions per row
    const int pg = p.bs_shift >= 0 ? (tc >> p.bs_shift) : tc / p.BS;
    const int slot = tc - pg * p.BS;
    return cache + (int64_t)pages_lds[pg] * page_stride * 2 + (int64_t)slot * row;
  };

  // accumulators of pass 3 (sixteen lanes per V row, one 16-byte piece each) and the running
  // softmax statistics; with CHUNKED the context is walked in slices of p.chunk tokens and both
  // are carried from slice to slice (rescaled when the maximum grows)
  const int g16 = tid >> 4, s16 = tid & 15;
  const bool onV = s16 < pieces;
  const int64_t offV = (int64_t)h * p.D * 2 + (onV ? s16 * 16 : 0);
  float acc[G][8], m_run[G], l_run[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m_run[g] = -INFINITY;
    l_run[g] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
  }
  auto slice = [&](const int c0, const int Tc) {   // Tc tokens from c0; LDS indices are slice-local
    // ---- pass 1: logits
    {
      u32x4 qa[G], qb[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const char* qp = p.q + (((int64_t)b * p.Hq + h * G + g) * p.D) * 2;
        qa[g] = onA ? *(const u32x4*)(qp + sub * 16) : zero4;
        qb[g] = onB ? *(const u32x4*)(qp + (sub + 8) * 16) : zero4;
      }
      // rows of the next trip are requested before the current ones are consumed
      u32x4 ka[kUnroll], kb[kUnroll], na[kUnroll], nb[kUnroll];
      auto fetch_k = [&](int t0, u32x4* a, u32x4* bq) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const char* base = row_base(p.k, p.k_sp, c0 + t0 + u * kGroups + grp);
          a[u] = ZP_DEC_LOAD((const u32x4*)(base + offA));
          bq[u] = ZP_DEC_LOAD((const u32x4*)(base + offB));
        }
      };
      fetch_k(0, ka, kb);
      for (int t0 = 0; t0 < Tc; t0 += kGroups * kUnroll) {
        const bool more = t0 + kGroups * kUnroll < Tc;
        if (more) fetch_k(t0 + kGroups * kUnroll, na, nb);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int t = t0 + u * kGroups + grp;
          float mine = 0.f;
#pragma unroll
          for (int g = 0; g < G; ++g) {
            float a = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) a = dot2<T>(ka[u][i], qa[g][i], a);
#pragma unroll
            for (int i = 0; i < 4; ++i) a = dot2<T>(kb[u][i], qb[g][i], a);
            a = group8_sum(a);
            mine = (sub == g) ? a : mine;
          }
          if (sub < G && t < Tc) logit[sub * Tpad + t] = mine * p.scale;
        }
        if (more) {
#pragma unroll
          for (int u = 0; u < kUnroll; ++u) { ka[u] = na[u]; kb[u] = nb[u]; }
        }
      }
    }
    __syncthreads();
    // ---- pass 2: softmax statistics per head, p packed in pairs (t, t + 32)
    {
      float mx[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float m = -INFINITY;
        for (int t = tid; t < Tc; t += kThreads) m = fmaxf(m, logit[g * Tpad + t]);
        m = wave_max(m);
        if (lane == 0) red[wave * G + g] = m;
      }
      __syncthreads();
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float m = red[g];
        for (int w = 1; w < kWaves; ++w) m = fmaxf(m, red[w * G + g]);
        mx[g] = CHUNKED ? fmaxf(m, m_run[g]) : m;
      }
      __syncthreads();
      const int npairs = ((Tc + 63) >> 6) * 32;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float s = 0.f;
        for (int pi = tid; pi < npairs; pi += kThreads) {
          const int t = (pi >> 5) * 64 + (pi & 31);
          // each token belongs to exactly one pair, so the packed word can overwrite logit[t]
          const float e0 = t < Tc ? __expf(logit[g * Tpad + t] - mx[g]) : 0.f;
          const float e1 = t + 32 < Tc ? __expf(logit[g * Tpad + t + 32] - mx[g]) : 0.f;
          s += e0 + e1;
          pw[g * Tpad + t] = pack2<T>(e0, e1);
        }
        s = wave_sum(s);
        if (lane == 0) red[wave * G + g] = s;
      }
      __syncthreads();
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float s = 0.f;
        for (int w = 0; w < kWaves; ++w) s += red[w * G + g];
        if (CHUNKED) {
          // earlier slices were accumulated against a smaller maximum: bring them to this one
          const float f = __expf(m_run[g] - mx[g]);   // exp(-inf) = 0 on the first slice
          l_run[g] = l_run[g] * f + s;
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[g][i] *= f;
        } else {
          l_run[g] = s;
        }
        m_run[g] = mx[g];
      }
    }
    // ---- pass 3: P.V, two tokens per dot2; a trip covers two 64-token blocks, and row group
    // `g16` takes the pairs j = g16 and j = g16 + 16 of each.
    {
      constexpr int kPairs = 4;
      u32x4 vx[kPairs], vy[kPairs], nx[kPairs], ny[kPairs];
      auto fetch_v = [&](int t0, u32x4* x, u32x4* y) {
#pragma unroll
        for (int u = 0; u < kPairs; ++u) {
          const int t = c0 + t0 + (u >> 1) * 64 + (u & 1) * 16 + g16;
          x[u] = ZP_DEC_LOAD((const u32x4*)(row_base(p.v, p.v_sp, t) + offV));
          y[u] = ZP_DEC_LOAD((const u32x4*)(row_base(p.v, p.v_sp, t + 32) + offV));
        }
      };
      fetch_v(0, vx, vy);
      for (int t0 = 0; t0 < Tc; t0 += 16 * kPairs * 2) {
        const bool more = t0 + 16 * kPairs * 2 < Tc;
        if (more) fetch_v(t0 + 16 * kPairs * 2, nx, ny);
#pragma unroll
        for (int u = 0; u < kPairs; ++u) {
          const int t = t0 + (u >> 1) * 64 + (u & 1) * 16 + g16;  // partner is t + 32
          if (t < Tc) {
            uint32_t pp[G];
#pragma unroll
            for (int g = 0; g < G; ++g) pp[g] = pw[g * Tpad + t];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const uint32_t lo = __builtin_amdgcn_perm(vy[u][i], vx[u][i], 0x05040100u);  // (x.lo16, y.lo16)
              const uint32_t hi = __builtin_amdgcn_perm(vy[u][i], vx[u][i], 0x07060302u);  // (x.hi16, y.hi16)
#pragma unroll
              for (int g = 0; g < G; ++g) {
                acc[g][2 * i] = dot2<T>(lo, pp[g], acc[g][2 * i]);
                acc[g][2 * i + 1] = dot2<T>(hi, pp[g], acc[g][2 * i + 1]);
              }
            }
          }
        }
        if (more) {
#pragma unroll
          for (int u = 0; u < kPairs; ++u) { vx[u] = nx[u]; vy[u] = ny[u]; }
        }
      }
    }
  };
  if constexpr (CHUNKED) {
    for (int c0 = 0; c0 < Tn; c0 += p.chunk) {
      slice(c0, min(p.chunk, Tn - c0));
      __syncthreads();   // the next slice's logits overwrite this slice's p
    }
  } else {
    if (Tn > 0) slice(0, Tn);   // one pass: nothing is carried, the accumulators start at pass 3
  }
  float inv[G];
#pragma unroll
  for (int g = 0; g < G; ++g) inv[g] = l_run[g] > 0.f ? 1.f / l_run[g] : 0.f;
  // sum the 4 row groups of each wave (lanes with equal piece), then the waves through LDS
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float v = acc[g][i];
      v += lane_xor16(v);
      v += lane_xor32(v);
      acc[g][i] = v;
    }
  __syncthreads();  // p no longer needed: reuse the LDS
  float* part = lds;  // [kWaves][G][128]
  if (lane < 16) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < 8; ++i) part[(wave * G + g) * 128 + s16 * 8 + i] = acc[g][i];
  }
  __syncthreads();
  for (int e = tid; e < G * p.D; e += kThreads) {
    const int g = e / p.D, d = e - g * p.D;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) s += part[(w * G + g) * 128 + d];
    Elem<T>::st(p.out, ((int64_t)b * p.Hq + h * G + g) * p.D + d, s * inv[g]);
  }
}

// Contexts whose logits fit 72 KB of LDS (4608 tokens at a group of 4) run in one slice; longer
// ones (a long prompt before its first compression) are walked in slices of 2048 tokens.
constexpr int kSingleSliceBytes = 72 * 1024;
constexpr int kSliceTokens = 2048;

template <typename T, int G>
int launch_decode(DecodeArgs a, hipStream_t st) {
  const int Tpad = (a.NB * a.BS + 63) & ~63;
  const size_t part = sizeof(float) * kWaves * G * 128;
  const bool chunked = sizeof(float) * (size_t)G * Tpad > kSingleSliceBytes;
  a.chunk = chunked ? kSliceTokens : 0;
  size_t smem = sizeof(float) * (size_t)G * (chunked ? kSliceTokens : Tpad);
  if (part > smem) smem = part;
  const void* fn = chunked ? (const void*)paged_decode_kernel<T, G, true>
                           : (const void*)paged_decode_kernel<T, G, false>;
  if (smem > 64 * 1024 &&
      hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    zp_set_error("paged_decode_attention: cannot reserve %zu bytes of LDS", smem);
    return ZP_EHIP;
  }
  const dim3 grid((unsigned)(a.B * a.Hkv));
  if (chunked) hipLaunchKernelGGL((paged_decode_kernel<T, G, true>), grid, dim3(kThreads), smem, st, a);
  else hipLaunchKernelGGL((paged_decode_kernel<T, G, false>), grid, dim3(kThreads), smem, st, a);
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
  ZP_REQUIRE(NB <= kMaxTablePages, "paged_decode_attention: more than %d table entries", kMaxTablePages);
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
  a.bs_shift = -1;
  if ((BS & (BS - 1)) == 0)
    for (a.bs_shift = 0; (1 << a.bs_shift) < BS; ++a.bs_shift) {}
  hipStream_t st = (hipStream_t)stream;
  if (dtype == ZP_BF16) return dispatch_group<BF16>(a, st);
  return dispatch_group<F16>(a, st);
}
