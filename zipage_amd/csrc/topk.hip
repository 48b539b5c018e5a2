// Per-row top-k keep mask by radix select (one workgroup per row).
//
// Scores are mapped to order-preserving 32-bit keys.  The k-th largest key v* is found by a
// radix select over 8-bit digits, most significant first (block_radix_select: LDS digit
// histograms, a wave-level suffix scan over the bins, one barrier per pass); 16-bit inputs
// only need the upper 16 (bf16: two passes) or 19 (fp16: three) bits.  Every key > v* is kept; of the keys
// equal to v*, the k - count(>v*) with the LOWEST indices are kept, which a block-wide
// exclusive scan over index-ordered per-thread chunks decides.
#include "common.h"
#include <limits.h>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kHistCopies = 4;   // copies of the radix-select digit bins (see block_radix_select)

// `low_bit`: the float image of this dtype has all bits below it clear; the key keeps them
// clear too (for negatives the complement would set them), so the bit search can stop there.
__device__ __forceinline__ uint32_t score_key(float f, int low_bit) {
  // selects only: this runs once per token inside straight-line code
  const uint32_t u = __float_as_uint(f);
  const uint32_t keep = 0xffffffffu << low_bit;
  uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  key = u == 0x80000000u ? 0x80000000u : key;                  // -0 == +0
  key = (u & 0x7fffffffu) > 0x7f800000u ? 0xffffffffu : key;   // NaN sorts largest
  return key & keep;
}

// Bits of the fp32 image below which this dtype's keys are all zero.
template <typename T> struct LowBit;
template <> struct LowBit<BF16> { static constexpr int v = 16; };
template <> struct LowBit<F16> { static constexpr int v = 13; };
template <> struct LowBit<F32> { static constexpr int v = 0; };

// Radix-select passes of a dtype and the digit histograms they rotate through.
template <int LOW> struct RadixPlan {
  static constexpr int passes = (32 - LOW + 7) / 8;
  static constexpr int buffers = passes < 3 ? passes : 3;
  static constexpr int words = buffers * 256 * kHistCopies;
};

// Zero the digit histograms; a barrier must follow before block_radix_select is entered.
template <int LOW>
__device__ __forceinline__ void radix_select_prepare(int* hist) {
#pragma unroll
  for (int c = 0; c < RadixPlan<LOW>::words / kThreads; ++c) hist[c * kThreads + threadIdx.x] = 0;
}

// k-th largest key of a row held by the 256 threads of a workgroup, by radix select: 8 bits per
// pass, most significant digit first.  Every thread adds the digit of each of its keys that still
// matches the prefix to a 256-bin LDS histogram (fire-and-forget adds, no dependent chain); every
// wave then reads the bins (four per lane, highest digits in lane 0), finds the bin that holds the
// k-th largest key with a prefix sum over its lanes (DPP adds), and the search descends into that
// bin.  All waves compute the same digit from the same bins, so one barrier per pass suffices: bf16
// keys take two passes, fp16 three, and each pass has its own bins, zeroed up front; fp32 keys take
// four and the last pass reuses the first one's bins, cleared during the third pass (they were last
// read before the second pass's barrier).  `each(f)` calls
// f(key) for every key of the calling thread.  Expects radix_select_prepare() and a barrier.
// Returns the k-th largest key; `n_gt` receives the number of keys strictly above it.
template <int LOW, typename Each>
__device__ __forceinline__ uint32_t block_radix_select(Each each, int k, int* hist /* [buffers][256][kHistCopies] */,
                                                       int& n_gt) {
  const int tid = threadIdx.x, lane = tid & 63;
  uint32_t prefix = 0;
  int kk = k;
  n_gt = 0;
  if (k <= 0) return 0xffffffffu;            // above every key: nothing is kept
  constexpr int HB = kHistCopies * 256;
  // scores cluster in a few exponents, so most lanes of a wave hit the same few bins and LDS adds
  // to one address serialise: lane l adds to copy l % kHistCopies of the bins.  The copies of one
  // bin are adjacent words, i.e. they sit in different LDS banks (copies 256 words apart would all
  // share the bank of their bin and serialise just the same).
  int* mycopy = hist + (lane % kHistCopies);
  const int dbase = 4 * (63 - lane);         // this lane's four bins: digits dbase .. dbase + 3
  int pp = 0;
#pragma unroll
  for (int sh = 24; sh + 8 > LOW; sh -= 8) {
    int* cur = hist + pp * HB;
    const int nx = pp == 2 ? 0 : pp + 1;
    if (sh == 8 && LOW < 8) {                // a fourth pass follows: it reuses the first pass's bins
#pragma unroll
      for (int c = 0; c < HB / kThreads; ++c) hist[nx * HB + c * kThreads + tid] = 0;
    }
    const uint32_t hi_mask = sh == 24 ? 0u : (0xffffffffu << (sh + 8));
    each([&](uint32_t key) {
      if (sh == 24 || (key & hi_mask) == prefix)
        atomicAdd(&mycopy[pp * HB + ((key >> sh) & 0xff) * kHistCopies], 1);
    });
    __syncthreads();
    // this lane's 4 bins x kHistCopies copies are 4 * kHistCopies consecutive words
    int e[4 * kHistCopies];
#pragma unroll
    for (int c = 0; c < kHistCopies; ++c) {
      const int4 o = *(const int4*)(cur + dbase * kHistCopies + 4 * c);
      e[4 * c] = o.x; e[4 * c + 1] = o.y; e[4 * c + 2] = o.z; e[4 * c + 3] = o.w;
    }
    int bv[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int t = e[q * kHistCopies];
#pragma unroll
      for (int c = 1; c < kHistCopies; ++c) t += e[q * kHistCopies + c];
      bv[q] = t;
    }
    int4 bins = make_int4(bv[0], bv[1], bv[2], bv[3]);
    const int mine = bins.x + bins.y + bins.z + bins.w;
    const int inc = wave_prefix_sum_incl(mine);   // keys with a digit >= dbase
    const int above = inc - mine;                  // keys in the bins of lower lanes (higher digits)
    const bool here = above < kk && kk <= inc;
    int digit = 0, over = 0;
    if (here) {
      int acc = above;
      digit = -1;
#pragma unroll
      for (int q = 3; q >= 0; --q) {
        if (digit < 0) {
          if (acc + bv[q] >= kk) { digit = dbase + q; over = acc; }
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

// Exclusive rank of this thread's `count` among the workgroup's threads in index order.
__device__ __forceinline__ int block_exclusive_rank(int count, int* scan_lds) {
  const int inc = wave_prefix_sum_incl(count);
  if (lane_id() == 63) scan_lds[wave_id()] = inc;
  __syncthreads();
  int rank = inc - count;
  for (int i = 0; i < wave_id(); ++i) rank += scan_lds[i];
  return rank;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void topk_mask_kernel(const void* __restrict__ scores,
                                                             uint8_t* __restrict__ flag, int Tn,
                                                             int k, int low_bit) {
  extern __shared__ uint32_t keys[];
  __shared__ __align__(16) int hist[RadixPlan<LowBit<T>::v>::words];
  __shared__ int scan_lds[kWaves];
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * Tn;
  for (int t = tid; t < Tn; t += kThreads) keys[t] = score_key(Elem<T>::ld(scores, base + t), low_bit);
  radix_select_prepare<LowBit<T>::v>(hist);
  __syncthreads();

  int n_gt;
  const uint32_t prefix = block_radix_select<LowBit<T>::v>(
      [&](auto f) { for (int t = tid; t < Tn; t += kThreads) f(keys[t]); }, k, hist, n_gt);
  const int need_eq = k - n_gt;  // >= 1 whenever 1 <= k <= Tn

  // index-ordered pass
  const int chunk = (Tn + kThreads - 1) / kThreads;
  const int s0 = min(tid * chunk, Tn), s1 = min(s0 + chunk, Tn);
  int ce = 0;
  for (int s = s0; s < s1; ++s) ce += keys[s] == prefix ? 1 : 0;
  int rank = block_exclusive_rank(ce, scan_lds);
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

// Rows of at most 256 * PER tokens, pages of at least PER tokens and a pooling window of at most
// 7: every thread owns a contiguous, index-ordered chunk of PER tokens (which therefore touches at
// most two pages), reads the PER + 6 raw scores its windows cover from LDS once and keeps its keys
// in registers.  The row sits in LDS between runs of the pooling's neutral value, so no window
// read is bounds-checked; the pooling variant (POOLK: 0 none, 1..3 max pooling of half-width POOLK,
// -1 average) and the presence of a redundancy row (RED) are compile-time, so a thread's tokens
// are straight-line code.
constexpr int kSelHalf = 3;
constexpr int kSelPad = 4;   // floats in front of the row (keeps it 16-byte aligned)
template <typename T, int PER, int POOLK, bool RED>
__global__ __launch_bounds__(kThreads) void select_reg_kernel(SelectArgs p) {
  extern __shared__ float sel_smem[];
  __shared__ __align__(16) int hist[RadixPlan<LowBit<T>::v>::words];
  __shared__ int scan_lds[kWaves];
  __shared__ float max_lds[kWaves];
  const int tid = threadIdx.x;
  const int Tn = p.NB * p.BS;
  const uint32_t r = blockIdx.x;          // 32-bit: a 64-bit division costs hundreds of scalar instructions
  const int b = (int)((r / (uint32_t)p.Hkv) % (uint32_t)p.B);
  const int64_t base = (int64_t)r * Tn;
  float* row = sel_smem + kSelPad;                    // row[-kSelHalf .. Tn + PER + kSelHalf)
  int* trow = (int*)(row + Tn + PER + kSelPad);       // the sequence's page codes, then two pads

  // every global read of the prologue is issued before the first wait
  const uint8_t was_compressed = p.compressed[b];
  for (int i = tid; i < p.NB + 2; i += kThreads) trow[i] = i < p.NB ? p.table[(int64_t)b * p.NB + i] : -1;
  stage_row<T>(p.scores, base, Tn, row);
  {
    const float neutral = POOLK > 0 ? -INFINITY : 0.f;
    if (tid < kSelPad) row[tid - kSelPad] = neutral;
    else if (tid < 2 * kSelPad + PER) row[Tn + tid - kSelPad] = neutral;
  }
  radix_select_prepare<LowBit<T>::v>(hist);
  float rmax = 1.f;
  if (RED && p.norm_r) {
    float m = -INFINITY;
    for (int t = tid; t < Tn; t += kThreads) m = fmaxf(m, Elem<T>::ld(p.red, base + t));
    rmax = block_max_of(m, max_lds);  // its barrier also publishes row[], trow[] and the bins
  } else {
    __syncthreads();
  }

  const int chunk = (Tn + kThreads - 1) / kThreads;  // <= PER <= BS
  const int s0 = min(tid * chunk, Tn), s1 = min(s0 + chunk, Tn);
  const bool pooled = POOLK != 0 && p.ksize > 1 && (p.continues || was_compressed == 0);
  // the (at most two) pages of this thread's tokens: [.., bnd) is page j0, [bnd, ..) page j0 + 1
  const int j0 = s0 / p.BS, bnd = (j0 + 1) * p.BS;
  const int code0 = trow[j0], code1 = trow[j0 + 1];
  // window tail of a last page, as a range of row indices (empty: starts at INT_MAX)
  const int wlo0 = (p.window > 0 && page_is_last(code0)) ? bnd - p.window : INT_MAX;
  const int wlo1 = (p.window > 0 && page_is_last(code1)) ? bnd + p.BS - p.window : INT_MAX;
  const bool pad0 = p.mask_pad && page_is_pad(code0), pad1 = p.mask_pad && page_is_pad(code1);

  float win[PER + 2 * kSelHalf];
#pragma unroll
  for (int j = 0; j < PER + 2 * kSelHalf; ++j) win[j] = row[s0 - kSelHalf + j];
  float rv[RED ? PER : 1];
  if constexpr (RED) {
#pragma unroll
    for (int i = 0; i < PER; ++i) rv[i] = Elem<T>::ld(p.red, base + min(s0 + i, Tn - 1));
  }
  float val[PER];
  uint32_t kreg[PER];
  // selects only, no short-circuit conditions: ten tokens of straight-line code per thread
  auto finish = [&](int i, float v) {
    const int t = s0 + i;
    if constexpr (RED) {
      float q = rv[i];
      if (p.norm_r) q = Elem<T>::rnd(q / rmax);
      const float a = Elem<T>::rnd(v * p.lam);
      const float c = Elem<T>::rnd(q * p.one_minus_lam);
      v = Elem<T>::rnd(a - c);
    }
    const bool first = t < bnd;
    const bool to_inf = (t < p.sink_len) | ((t >= wlo0) & first) | (t >= wlo1);
    const bool to_ninf = first ? pad0 : pad1;
    v = to_inf ? INFINITY : v;
    v = to_ninf ? -INFINITY : v;
    val[i] = v;
    const uint32_t key = score_key(v, LowBit<T>::v);
    kreg[i] = t < s1 ? key : 0u;   // 0: below every real key
  };
  if (pooled) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      float v = win[i + kSelHalf];
      if constexpr (POOLK > 0) {
#pragma unroll
        for (int d = 1; d <= POOLK; ++d) v = fmaxf(fmaxf(v, win[i + kSelHalf - d]), win[i + kSelHalf + d]);
      } else if constexpr (POOLK < 0) {
        const int half = p.ksize / 2;
        float acc = 0.f;  // ascending index order, as pool_kernel adds
#pragma unroll
        for (int d = -kSelHalf; d <= kSelHalf; ++d) {
          if (d >= -half && d <= half) acc += win[i + kSelHalf + d];
        }
        v = Elem<T>::rnd(acc / (float)p.ksize);
      }
      finish(i, v);
    }
  } else {
#pragma unroll
    for (int i = 0; i < PER; ++i) finish(i, win[i + kSelHalf]);
  }
  if (p.scores_out) {
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (s0 + i < s1) Elem<T>::st(p.scores_out, base + s0 + i, val[i]);
  }

  int n_gt;
  const uint32_t prefix = block_radix_select<LowBit<T>::v>(
      [&](auto f) {
#pragma unroll
        for (int i = 0; i < PER; ++i) f(kreg[i]);
      },
      p.k, hist, n_gt);
  // prefix is the k-th largest key; keep everything above it and the first few equal to it
  const int need_eq = p.k - n_gt;
  int ce = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) ce += (s0 + i < s1 && kreg[i] == prefix) ? 1 : 0;
  int rank = block_exclusive_rank(ce, scan_lds);  // its barrier: every thread has finished reading row[]
  uint8_t fb[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    uint8_t f = kreg[i] > prefix ? 1 : 0;
    if (kreg[i] == prefix) { f = rank < need_eq ? 1 : 0; ++rank; }
    fb[i] = f;
  }
  // a thread's flags are contiguous in the output: stored from registers, two per store when the
  // chunks start and end on even indices (the row base is then even as well)
  uint8_t* out = p.flag + base + s0;
  if (((chunk | Tn) & 1) == 0 && ((uintptr_t)p.flag & 1) == 0) {
#pragma unroll
    for (int i = 0; i + 1 < PER; i += 2)
      if (s0 + i < s1) *(uint16_t*)(out + i) = (uint16_t)(fb[i] | (fb[i + 1] << 8));
  } else {
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (s0 + i < s1) out[i] = fb[i];
  }
}

// Any row that fits LDS twice (raw scores + keys), any odd pooling window.
template <typename T>
__global__ __launch_bounds__(kThreads) void select_lds_kernel(SelectArgs p) {
  extern __shared__ float row[];
  __shared__ __align__(16) int hist[RadixPlan<LowBit<T>::v>::words];
  __shared__ int scan_lds[kWaves];
  __shared__ float max_lds[kWaves];
  const int tid = threadIdx.x;
  const int Tn = p.NB * p.BS;
  uint32_t* keys = (uint32_t*)(row + Tn);
  const uint32_t r = blockIdx.x;          // 32-bit: a 64-bit division costs hundreds of scalar instructions
  const int b = (int)((r / (uint32_t)p.Hkv) % (uint32_t)p.B);
  const int64_t base = (int64_t)r * Tn;
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
  radix_select_prepare<LowBit<T>::v>(hist);
  __syncthreads();

  const int chunk = (Tn + kThreads - 1) / kThreads;
  const int s0 = min(tid * chunk, Tn), s1 = min(s0 + chunk, Tn);
  int n_gt;
  const uint32_t prefix = block_radix_select<LowBit<T>::v>(
      [&](auto f) { for (int s = s0; s < s1; ++s) f(keys[s]); }, p.k, hist, n_gt);
  const int need_eq = p.k - n_gt;
  int ce = 0;
  for (int s = s0; s < s1; ++s) ce += keys[s] == prefix ? 1 : 0;
  int rank = block_exclusive_rank(ce, scan_lds);
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
  constexpr int PER = 10;
  const bool in_regs = Tn <= PER * kThreads && BS >= PER && pool_kernel_size <= 2 * kSelHalf + 1;
  const size_t smem = in_regs ? ((size_t)Tn + PER + 2 * kSelPad + NB + 2) * 4 : (size_t)Tn * 8;
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
#define ZP_SELECT_REG(POOLK)                                                                      \
  do {                                                                                            \
    if (redundancy) ZP_SELECT_LAUNCH((select_reg_kernel<T, PER, POOLK, true>));                   \
    else ZP_SELECT_LAUNCH((select_reg_kernel<T, PER, POOLK, false>));                             \
  } while (0)
#define ZP_SELECT_REG_ALL()                                                                       \
  do {                                                                                            \
    if (pool_kernel_size <= 1) ZP_SELECT_REG(0);                                                  \
    else if (pool_mode != ZP_POOL_MAX) ZP_SELECT_REG(-1);                                         \
    else if (pool_kernel_size == 3) ZP_SELECT_REG(1);                                             \
    else if (pool_kernel_size == 5) ZP_SELECT_REG(2);                                             \
    else ZP_SELECT_REG(3);                                                                        \
  } while (0)
  if (in_regs) {
    ZP_DISPATCH_DTYPE(dtype, ZP_SELECT_REG_ALL());
  } else {
    ZP_DISPATCH_DTYPE(dtype, ZP_SELECT_LAUNCH((select_lds_kernel<T>)));
  }
#undef ZP_SELECT_REG_ALL
#undef ZP_SELECT_REG
#undef ZP_SELECT_LAUNCH
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}
