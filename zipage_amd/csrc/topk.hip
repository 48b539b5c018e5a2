// Per-row top-k keep mask by radix select (one workgroup per row).
//
// Scores are mapped to order-preserving 32-bit keys.  The k-th largest key v* is found by a
// radix select over 8-bit digits, most significant first (block_radix_select: LDS digit
// histograms, a wave-level suffix scan over the bins, one barrier per pass); 16-bit inputs
// only need the upper 16 (bf16: two passes) or 19 (fp16: three) bits.  Every key > v* is kept; of the keys
// equal to v*, the k - count(>v*) with the LOWEST indices are kept, which a block-wide
// exclusive scan over index-ordered per-thread chunks decides.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kHistCopies = 8;   // copies of the radix-select digit bins (see block_radix_select)

// `low_bit`: the float image of this dtype has all bits below it clear; the key keeps them
// clear too (for negatives the complement would set them), so the bit search can stop there.
__device__ __forceinline__ uint32_t score_key(float f, int low_bit) {
  uint32_t u = __float_as_uint(f);
  const uint32_t keep = 0xffffffffu << low_bit;
  if ((u & 0x7fffffffu) > 0x7f800000u) return keep;  // NaN sorts largest
  if (u == 0x80000000u) u = 0u;                      // -0 == +0
  return ((u & 0x80000000u) ? ~u : (u | 0x80000000u)) & keep;
}

// k-th largest key of a row held by the 256 threads of a workgroup, by radix select: 8 bits per
// pass, most significant digit first.  Every thread adds the digit of each of its keys that still
// matches the prefix to a 256-bin LDS histogram (fire-and-forget adds, no dependent chain); every
// wave then reads the bins (four per lane), finds the bin that holds the k-th largest key with a
// suffix scan over its lanes, and the search descends into that bin.  All waves compute the same
// digit from the same bins, so one barrier per pass suffices (the bins rotate through three
// buffers: the one cleared during a pass was last read two passes ago, with a barrier between).  bf16 keys take two passes,
// fp16 three, fp32 four.  `each(f)` calls f(key) for every key of the calling thread.
// Returns the k-th largest key; `n_gt` receives the number of keys strictly above it.
template <typename Each>
__device__ __forceinline__ uint32_t block_radix_select(Each each, int k, int low_bit, int* hist /* [3][kHistCopies][256] */,
                                                       int& n_gt) {
  const int tid = threadIdx.x, lane = tid & 63;
  uint32_t prefix = 0;
  int kk = k;
  n_gt = 0;
  if (k <= 0) return 0xffffffffu;            // above every key: nothing is kept
  constexpr int HB = kHistCopies * 256;
#pragma unroll
  for (int c = 0; c < kHistCopies; ++c) hist[c * 256 + tid] = 0;   // kThreads == 256 bins
  __syncthreads();
  int pp = 0;
  // scores cluster in a few exponents, so most lanes of a wave hit the same few bins and LDS adds
  // to one address serialise: lane l adds to copy l % kHistCopies of the bins
  int* mycopy = hist + (lane % kHistCopies) * 256;
  for (int sh = 24; sh + 8 > low_bit; sh -= 8) {
    int* cur = hist + pp * HB;
    const int nx = pp == 2 ? 0 : pp + 1;
#pragma unroll
    for (int c = 0; c < kHistCopies; ++c)
      hist[nx * HB + c * 256 + tid] = 0;     // the next pass's bins (last read two passes ago)
    const uint32_t hi_mask = sh == 24 ? 0u : (0xffffffffu << (sh + 8));
    each([&](uint32_t key) {
      if ((key & hi_mask) == prefix) atomicAdd(&mycopy[pp * HB + ((key >> sh) & 0xff)], 1);
    });
    __syncthreads();
    int4 bins = *(const int4*)(cur + 4 * lane);
#pragma unroll
    for (int c = 1; c < kHistCopies; ++c) {
      const int4 o = *(const int4*)(cur + c * 256 + 4 * lane);
      bins.x += o.x; bins.y += o.y; bins.z += o.z; bins.w += o.w;
    }
    const int mine = bins.x + bins.y + bins.z + bins.w;
    int suf = mine;                          // inclusive suffix sum over the lanes (higher digits)
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_down(suf, o, 64);
      if (lane + o < 64) suf += t;
    }
    const int above = suf - mine;            // keys in the bins of higher lanes
    const bool here = above < kk && kk <= suf;
    int digit = 0, over = 0;
    if (here) {
      const int bv[4] = {bins.x, bins.y, bins.z, bins.w};
      int acc = above;
      digit = -1;
#pragma unroll
      for (int q = 3; q >= 0; --q) {
        if (digit < 0) {
          if (acc + bv[q] >= kk) { digit = 4 * lane + q; over = acc; }
          else acc += bv[q];
        }
      }
    }
    const unsigned long long who = __builtin_amdgcn_ballot_w64(here);
    const int src = who ? __builtin_ctzll(who) : 0;   // exactly one lane when k <= row length
    digit = __builtin_amdgcn_readlane(digit, src);
    over = __builtin_amdgcn_readlane(over, src);
    prefix |= (uint32_t)digit << sh;
    n_gt += over;
    kk -= over;
    pp = nx;
  }
  return prefix;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void topk_mask_kernel(const void* __restrict__ scores,
                                                             uint8_t* __restrict__ flag, int Tn,
                                                             int k, int low_bit) {
  extern __shared__ uint32_t keys[];
  __shared__ __align__(16) int hist[3][kHistCopies][256];
  __shared__ int scan_lds[kWaves];
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * Tn;
  for (int t = tid; t < Tn; t += kThreads) keys[t] = score_key(Elem<T>::ld(scores, base + t), low_bit);
  __syncthreads();

  int n_gt;
  const uint32_t prefix = block_radix_select(
      [&](auto f) { for (int t = tid; t < Tn; t += kThreads) f(keys[t]); }, k, low_bit, &hist[0][0][0], n_gt);
  const int need_eq = k - n_gt;  // >= 1 whenever 1 <= k <= Tn

  // index-ordered pass
  const int chunk = (Tn + kThreads - 1) / kThreads;
  const int s0 = min(tid * chunk, Tn), s1 = min(s0 + chunk, Tn);
  int ce = 0;
  for (int s = s0; s < s1; ++s) ce += keys[s] == prefix ? 1 : 0;
  // block-wide exclusive scan of ce
  int inc = ce;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int t = __shfl_up(inc, o, 64);
    if (lane_id() >= o) inc += t;
  }
  if (lane_id() == 63) scan_lds[wave_id()] = inc;
  __syncthreads();
  int rank = inc - ce;
  for (int i = 0; i < wave_id(); ++i) rank += scan_lds[i];
  for (int s = s0; s < s1; ++s) {
    const uint32_t key = keys[s];
    uint8_t f = 0;
    if (key > prefix) f = 1;
    else if (key == prefix) { f = rank < need_eq ? 1 : 0; ++rank; }
    flag[base + s] = f;
  }
}


// ------------------------------------------------------------------ fused selection
// Pooling, redundancy combine, sink / window / pad masks and the top-k of one score row in a
// single pass.  The per-element arithmetic and its rounding points are those of pool_kernel
// and epilogue_kernel, so the result equals running the three stages one after the other.
struct SelectArgs {
  const void* scores;
  void* scores_out;         // may be null
  const void* red;          // may be null
  uint8_t* flag;
  const int32_t* table;
  const uint8_t* compressed;
  int B, NB, BS, Hkv, ksize, continues, mode, norm_r;
  float lam, one_minus_lam;
  int sink_len, window, mask_pad, k, low_bit;
};

// Row -> LDS as fp32, 16 bytes per thread per step when the row allows it.
template <typename T>
__device__ __forceinline__ void stage_row(const void* __restrict__ src, int64_t base, int Tn,
                                          float* __restrict__ row) {
  constexpr int EPV = 16 / T::bytes;  // elements per 16-byte piece
  const char* p = (const char*)src + base * T::bytes;
  if ((Tn % EPV) == 0 && ((uintptr_t)p & 15) == 0) {
    for (int c = threadIdx.x; c < Tn / EPV; c += kThreads) {
      const vec16 v = ((const vec16*)p)[c];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      float* dst = row + c * EPV;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (T::bytes == 4) {
          dst[i] = __uint_as_float(w[i]);
        } else {
          const uint16_t lo = (uint16_t)(w[i] & 0xffffu), hi = (uint16_t)(w[i] >> 16);
          dst[2 * i] = Elem<T>::ld(&lo, 0);
          dst[2 * i + 1] = Elem<T>::ld(&hi, 0);
        }
      }
    }
  } else {
    for (int t = threadIdx.x; t < Tn; t += kThreads) row[t] = Elem<T>::ld(src, base + t);
  }
}

__device__ __forceinline__ float block_max_of(float m, float* max_lds) {
  m = wave_max(m);
  if (lane_id() == 0) max_lds[wave_id()] = m;
  __syncthreads();
  float r = max_lds[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) r = fmaxf(r, max_lds[i]);
  return r;
}

// Combine with the redundancy and apply the masks to one pooled value (epilogue_kernel's
// per-element body).
template <typename T>
__device__ __forceinline__ float select_finish(const SelectArgs& p, float v, int t, int64_t base,
                                               int code, int slot, float rmax) {
  if (p.red) {
    float rv = Elem<T>::ld(p.red, base + t);
    if (p.norm_r) rv = Elem<T>::rnd(rv / rmax);
    const float a = Elem<T>::rnd(v * p.lam);
    const float c = Elem<T>::rnd(rv * p.one_minus_lam);
    v = Elem<T>::rnd(a - c);
  }
  if (t < p.sink_len) v = INFINITY;
  if (p.window > 0 && page_is_last(code) && slot >= p.BS - p.window) v = INFINITY;
  if (p.mask_pad && page_is_pad(code)) v = -INFINITY;
  if (p.scores_out) Elem<T>::st(p.scores_out, base + t, v);
  return v;
}

// Flags staged in LDS by index-ordered owners, then written out coalesced.
__device__ __forceinline__ void write_flags(const uint8_t* fl, uint8_t* __restrict__ flag,
                                            int64_t base, int Tn) {
  if ((Tn & 3) == 0 && ((uintptr_t)flag & 3) == 0) {
    const uint32_t* src = (const uint32_t*)fl;
    uint32_t* dst = (uint32_t*)(flag + base);
    for (int t = threadIdx.x; t < Tn / 4; t += kThreads) dst[t] = src[t];
  } else {
    for (int t = threadIdx.x; t < Tn; t += kThreads) flag[base + t] = fl[t];
  }
}

// Rows of at most 256 * PER tokens with a pooling window of at most 7: every thread owns a
// contiguous, index-ordered chunk of PER tokens, reads the PER + 6 raw scores its windows
// cover from LDS once and keeps its keys in registers, so each step of the bit search is
// PER compares, one wave sum and one barrier.
constexpr int kSelHalf = 3;
template <typename T, int PER>
__global__ __launch_bounds__(kThreads) void select_reg_kernel(SelectArgs p) {
  extern __shared__ float row[];
  __shared__ __align__(16) int hist[3][kHistCopies][256];
  __shared__ int scan_lds[kWaves];
  __shared__ float max_lds[kWaves];
  const int tid = threadIdx.x;
  const int Tn = p.NB * p.BS;
  const int64_t r = blockIdx.x;
  const int b = (int)((r / p.Hkv) % p.B);
  const int64_t base = r * Tn;
  int* trow = (int*)(row + Tn);  // the sequence's page codes, NB words behind the row

  // every global read of the prologue is issued before the first wait
  const uint8_t was_compressed = p.compressed[b];
  for (int i = tid; i < p.NB; i += kThreads) trow[i] = p.table[(int64_t)b * p.NB + i];
  stage_row<T>(p.scores, base, Tn, row);
  float rmax = 1.f;
  if (p.red && p.norm_r) {
    float m = -INFINITY;
    for (int t = tid; t < Tn; t += kThreads) m = fmaxf(m, Elem<T>::ld(p.red, base + t));
    rmax = block_max_of(m, max_lds);  // its barrier also publishes row[] and trow[]
  } else {
    __syncthreads();
  }

  const int chunk = (Tn + kThreads - 1) / kThreads;  // <= PER
  const int s0 = min(tid * chunk, Tn), s1 = min(s0 + chunk, Tn);
  const bool pooled = p.ksize > 1 && (p.continues || was_compressed == 0);
  const int half = pooled ? p.ksize / 2 : 0;
  const bool is_max = p.mode == ZP_POOL_MAX;
  float win[PER + 2 * kSelHalf];
#pragma unroll
  for (int j = 0; j < PER + 2 * kSelHalf; ++j) {
    const int idx = s0 - kSelHalf + j;
    win[j] = (idx >= 0 && idx < Tn) ? row[idx] : (is_max ? -INFINITY : 0.f);
  }
  int j = s0 / p.BS, slot = s0 - j * p.BS;
  int code = s0 < Tn ? trow[j] : -1;
  uint32_t kreg[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    kreg[i] = 0u;  // below every real key
    if (s0 + i < s1) {
      float v = win[i + kSelHalf];
      if (pooled) {
        if (is_max) {
#pragma unroll
          for (int d = 1; d <= kSelHalf; ++d) {
            if (d <= half) v = fmaxf(fmaxf(v, win[i + kSelHalf - d]), win[i + kSelHalf + d]);
          }
        } else {
          float acc = 0.f;  // ascending index order, as pool_kernel adds
#pragma unroll
          for (int d = -kSelHalf; d <= kSelHalf; ++d) {
            if (d >= -half && d <= half) acc += win[i + kSelHalf + d];
          }
          v = Elem<T>::rnd(acc / (float)p.ksize);
        }
      }
      v = select_finish<T>(p, v, s0 + i, base, code, slot, rmax);
      kreg[i] = score_key(v, p.low_bit);
      if (++slot == p.BS) {
        slot = 0;
        ++j;
        if (s0 + i + 1 < s1) code = trow[j];
      }
    }
  }

  int n_gt;
  const uint32_t prefix = block_radix_select(
      [&](auto f) {
#pragma unroll
        for (int i = 0; i < PER; ++i) f(kreg[i]);
      },
      p.k, p.low_bit, &hist[0][0][0], n_gt);
  // prefix is the k-th largest key; keep everything above it and the first few equal to it
  const int need_eq = p.k - n_gt;
  int ce = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) ce += (s0 + i < s1 && kreg[i] == prefix) ? 1 : 0;
  int inc = ce;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int t = __shfl_up(inc, o, 64);
    if (lane_id() >= o) inc += t;
  }
  if (lane_id() == 63) scan_lds[wave_id()] = inc;
  __syncthreads();  // every thread has long finished reading row[] as floats
  int rank = inc - ce;
  for (int i = 0; i < wave_id(); ++i) rank += scan_lds[i];
  uint8_t* fl = (uint8_t*)row;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    if (s0 + i < s1) {
      uint8_t f = kreg[i] > prefix ? 1 : 0;
      if (kreg[i] == prefix) { f = rank < need_eq ? 1 : 0; ++rank; }
      fl[s0 + i] = f;
    }
  }
  __syncthreads();
  write_flags(fl, p.flag, base, Tn);
}

// Any row that fits LDS twice (raw scores + keys), any odd pooling window.
template <typename T>
__global__ __launch_bounds__(kThreads) void select_lds_kernel(SelectArgs p) {
  extern __shared__ float row[];
  __shared__ __align__(16) int hist[3][kHistCopies][256];
  __shared__ int scan_lds[kWaves];
  __shared__ float max_lds[kWaves];
  const int tid = threadIdx.x;
  const int Tn = p.NB * p.BS;
  uint32_t* keys = (uint32_t*)(row + Tn);
  const int64_t r = blockIdx.x;
  const int b = (int)((r / p.Hkv) % p.B);
  const int64_t base = r * Tn;
  const int32_t* trow = p.table + (int64_t)b * p.NB;

  stage_row<T>(p.scores, base, Tn, row);
  float rmax = 1.f;
  if (p.red && p.norm_r) {
    float m = -INFINITY;
    for (int t = tid; t < Tn; t += kThreads) m = fmaxf(m, Elem<T>::ld(p.red, base + t));
    rmax = block_max_of(m, max_lds);
  } else {
    __syncthreads();
  }

  const bool pooled = p.ksize > 1 && (p.continues || p.compressed[b] == 0);
  const int half = p.ksize / 2;
  for (int t = tid; t < Tn; t += kThreads) {
    float v = row[t];
    if (pooled) {
      const int lo = max(t - half, 0), hi = min(t + half, Tn - 1);
      if (p.mode == ZP_POOL_MAX) {
        v = row[lo];
        for (int i = lo + 1; i <= hi; ++i) v = fmaxf(v, row[i]);
      } else {
        float acc = 0.f;
        for (int i = lo; i <= hi; ++i) acc += row[i];
        v = Elem<T>::rnd(acc / (float)p.ksize);
      }
    }
    const int j = t / p.BS, slot = t - j * p.BS;
    v = select_finish<T>(p, v, t, base, trow[j], slot, rmax);
    keys[t] = score_key(v, p.low_bit);
  }
  __syncthreads();

  const int chunk = (Tn + kThreads - 1) / kThreads;
  const int s0 = min(tid * chunk, Tn), s1 = min(s0 + chunk, Tn);
  int n_gt;
  const uint32_t prefix = block_radix_select(
      [&](auto f) { for (int s = s0; s < s1; ++s) f(keys[s]); }, p.k, p.low_bit, &hist[0][0][0], n_gt);
  const int need_eq = p.k - n_gt;
  int ce = 0;
  for (int s = s0; s < s1; ++s) ce += keys[s] == prefix ? 1 : 0;
  int inc = ce;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int t = __shfl_up(inc, o, 64);
    if (lane_id() >= o) inc += t;
  }
  if (lane_id() == 63) scan_lds[wave_id()] = inc;
  __syncthreads();
  int rank = inc - ce;
  for (int i = 0; i < wave_id(); ++i) rank += scan_lds[i];
  uint8_t* fl = (uint8_t*)row;
  for (int s = s0; s < s1; ++s) {
    const uint32_t key = keys[s];
    uint8_t f = key > prefix ? 1 : 0;
    if (key == prefix) { f = rank < need_eq ? 1 : 0; ++rank; }
    fl[s] = f;
  }
  __syncthreads();
  write_flags(fl, p.flag, base, Tn);
}

}  // namespace

extern "C" int zp_topk_mask(const void* scores, uint8_t* flag_out, int32_t rows, int32_t Tn,
                            int32_t k, int32_t dtype, void* stream) {
  ZP_REQUIRE(rows >= 0 && Tn > 0, "topk_mask: bad dims rows=%d T=%d", rows, Tn);
  ZP_REQUIRE(k >= 0, "topk_mask: negative k");
  ZP_REQUIRE(k <= Tn, "topk_mask: k=%d out of range for a row of %d", k, Tn);
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "topk_mask: unknown dtype tag %d", dtype);
  ZP_REQUIRE((int64_t)Tn * 4 <= 150 * 1024, "topk_mask: row of %d tokens exceeds LDS", Tn);
  if (rows == 0) return ZP_OK;
  ZP_REQUIRE(scores && flag_out, "topk_mask: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const size_t smem = (size_t)Tn * 4;
  const int low_bit = dtype == ZP_BF16 ? 16 : (dtype == ZP_F16 ? 13 : 0);
#define ZP_TOPK_LAUNCH()                                                                          \
  do {                                                                                            \
    if (smem > 64 * 1024 &&                                                                       \
        hipFuncSetAttribute((const void*)topk_mask_kernel<T>,                                     \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) { \
      zp_set_error("topk_mask: cannot reserve %zu bytes of LDS", smem);                           \
      return ZP_EHIP;                                                                             \
    }                                                                                             \
    hipLaunchKernelGGL((topk_mask_kernel<T>), dim3(rows), dim3(kThreads), smem, st, scores,       \
                       flag_out, Tn, k, low_bit);                                                 \
  } while (0)
  ZP_DISPATCH_DTYPE(dtype, ZP_TOPK_LAUNCH());
#undef ZP_TOPK_LAUNCH
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

extern "C" int zp_select_topk(const void* scores, void* scores_out, const void* redundancy,
                              uint8_t* flag_out, const int32_t* block_table,
                              const uint8_t* compressed, int32_t L, int32_t B, int32_t NB,
                              int32_t BS, int32_t Hkv, int32_t pool_kernel_size,
                              int32_t continues_pooling, int32_t pool_mode, int32_t max_norm_red,
                              double redudancy_lambda, int32_t sink_len, int32_t window,
                              int32_t mask_pad, int32_t k, int32_t dtype, void* stream) {
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0, "select_topk: bad dims");
  const int64_t Tn = (int64_t)NB * BS;
  ZP_REQUIRE(k >= 0 && k <= Tn, "select_topk: k=%d out of range for a row of %lld", k, (long long)Tn);
  ZP_REQUIRE(pool_kernel_size <= 1 || (pool_kernel_size & 1),
             "select_topk: pooling kernel_size %d must be odd", pool_kernel_size);
  ZP_REQUIRE(pool_mode == ZP_POOL_MAX || pool_mode == ZP_POOL_AVG, "select_topk: unknown pooling mode %d",
             pool_mode);
  ZP_REQUIRE(window >= 0 && window <= BS, "select_topk: window %d outside [0, BS=%d]", window, BS);
  ZP_REQUIRE(sink_len >= 0, "select_topk: negative sink_len");
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "select_topk: unknown dtype tag %d", dtype);
  ZP_REQUIRE(Tn * 8 <= 150 * 1024, "select_topk: row of %lld tokens exceeds LDS", (long long)Tn);
  if (L == 0 || B == 0) return ZP_OK;
  ZP_REQUIRE(scores && flag_out && block_table && compressed, "select_topk: null pointer");
  hipStream_t st = (hipStream_t)stream;
  SelectArgs p;
  p.scores = scores; p.scores_out = scores_out; p.red = redundancy; p.flag = flag_out;
  p.table = block_table; p.compressed = compressed;
  p.B = B; p.NB = NB; p.BS = BS; p.Hkv = Hkv; p.ksize = pool_kernel_size;
  p.continues = continues_pooling; p.mode = pool_mode; p.norm_r = max_norm_red;
  p.lam = (float)redudancy_lambda; p.one_minus_lam = (float)(1.0 - redudancy_lambda);
  p.sink_len = sink_len; p.window = window; p.mask_pad = mask_pad; p.k = k;
  p.low_bit = dtype == ZP_BF16 ? 16 : (dtype == ZP_F16 ? 13 : 0);
  dim3 grid((unsigned)((int64_t)L * B * Hkv));
  const bool in_regs = Tn <= 10 * kThreads && pool_kernel_size <= 2 * kSelHalf + 1;
  const size_t smem = in_regs ? (size_t)Tn * 4 + (size_t)NB * 4 : (size_t)Tn * 8;
#define ZP_SELECT_LAUNCH(KERNEL)                                                                  \
  do {                                                                                            \
    if (smem > 64 * 1024 &&                                                                       \
        hipFuncSetAttribute((const void*)KERNEL, hipFuncAttributeMaxDynamicSharedMemorySize,      \
                            (int)smem) != hipSuccess) {                                           \
      zp_set_error("select_topk: cannot reserve %zu bytes of LDS", smem);                         \
      return ZP_EHIP;                                                                             \
    }                                                                                             \
    hipLaunchKernelGGL(KERNEL, grid, dim3(kThreads), smem, st, p);                                \
  } while (0)
  if (in_regs) {
    ZP_DISPATCH_DTYPE(dtype, ZP_SELECT_LAUNCH((select_reg_kernel<T, 10>)));
  } else {
    ZP_DISPATCH_DTYPE(dtype, ZP_SELECT_LAUNCH((select_lds_kernel<T>)));
  }
#undef ZP_SELECT_LAUNCH
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}
