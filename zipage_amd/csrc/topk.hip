// Per-row top-k keep mask by radix select (one workgroup per row).
//
// Scores are mapped to order-preserving 32-bit keys held in LDS.  The k-th largest key
// v* is found most-significant-bit first: a candidate bit is kept when at least k keys
// are >= the candidate prefix; each step is one block-wide count (ballot-free register
// counts, xor-shuffle wave sums, one barrier with ping-pong LDS slots).  16-bit inputs
// only need the upper 16 (bf16) or 19 (fp16) bits.  Every key > v* is kept; of the keys
// equal to v*, the k - count(>v*) with the LOWEST indices are kept, which a block-wide
// exclusive scan over index-ordered per-thread chunks decides.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

// `low_bit`: the float image of this dtype has all bits below it clear; the key keeps them
// clear too (for negatives the complement would set them), so the bit search can stop there.
__device__ __forceinline__ uint32_t score_key(float f, int low_bit) {
  uint32_t u = __float_as_uint(f);
  const uint32_t keep = 0xffffffffu << low_bit;
  if ((u & 0x7fffffffu) > 0x7f800000u) return keep;  // NaN sorts largest
  if (u == 0x80000000u) u = 0u;                      // -0 == +0
  return ((u & 0x80000000u) ? ~u : (u | 0x80000000u)) & keep;
}

__device__ __forceinline__ int block_count(int c, int* slots /* kWaves */) {
  c = wave_sum_i(c);
  if (lane_id() == 0) slots[wave_id()] = c;
  __syncthreads();
  int s = 0;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) s += slots[i];
  return s;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void topk_mask_kernel(const void* __restrict__ scores,
                                                             uint8_t* __restrict__ flag, int Tn,
                                                             int k, int low_bit) {
  extern __shared__ uint32_t keys[];
  __shared__ int slots[2][kWaves];
  __shared__ int scan_lds[kWaves];
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * Tn;
  for (int t = tid; t < Tn; t += kThreads) keys[t] = score_key(Elem<T>::ld(scores, base + t), low_bit);
  __syncthreads();

  uint32_t prefix = 0;
  int pp = 0;
  for (int bit = 31; bit >= low_bit; --bit) {
    const uint32_t cand = prefix | (1u << bit);
    int c = 0;
    for (int t = tid; t < Tn; t += kThreads) c += keys[t] >= cand ? 1 : 0;
    if (block_count(c, slots[pp]) >= k) prefix = cand;
    pp ^= 1;
  }
  // keys strictly above the threshold
  int cg = 0;
  for (int t = tid; t < Tn; t += kThreads) cg += keys[t] > prefix ? 1 : 0;
  const int n_gt = block_count(cg, slots[pp]);
  const int need_eq = k - n_gt;  // >= 1 whenever k <= Tn

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
