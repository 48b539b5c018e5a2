// Key-redundancy scores: cosine-similarity Gram matrix of cached keys, per page
// ("lightning") or over the whole sequence ("raw"), with the reference's claim rule:
// the diagonal is zeroed and, for every column, the LAST row whose similarity exceeds the
// threshold is zeroed too; the row sums are the redundancy logits.
//
// The Gram matrix is symmetric, so "last row over the threshold in column j" equals "last
// column over the threshold in row j" (the key's claim); the claimed entries are subtracted
// afterwards from the rows they were taken from:
//     r_i = sum_j S_ij  -  sum_{j : c*(j) = i} S_ji .
//
// Kernels in this file:
//   gram_kernel        fp32 caches, both variants, any page size and table length:
//                      v_mfma_f32_32x32x2_f32 on keys divided by their norm in fp32, full matrix,
//                      a wave owns 32 rows for all columns.
//   gram_page_f32_kernel  fp32 caches, lightning, pages of at most 256 keys: a workgroup walks the
//                      pages of a row; the normalised page resident in LDS as two fp16 planes per
//                      element (fp32-grade products on the 16-bit matrix instructions), one
//                      barrier, both operands read from that copy, every pair of key blocks once.
//   gram_raw_sym_f32_kernel  fp32 caches, raw, pages of at most 256 keys and tables of at most 16
//                      pages: every unordered pair of pages once, column tiles staged as the same
//                      two planes.
//   gram_split_kernel  16-bit caches, lightning with pages above 256 keys: normalised keys
//                      split into two bf16 planes, three MFMAs per k-step, full matrix.
//   gram_page_kernel   16-bit caches, lightning: a workgroup walks the pages of one (layer,
//                      sequence, kv head) row; stored keys loaded straight into LDS and put on
//                      the matrix cores, 1/norm factors on the accumulators, every pair of key
//                      blocks once, the summed key as a product over the keys, the next page
//                      requested while a page's row sums are finished.
//   raw_prep_kernel, gram_raw_wide_kernel / gram_raw_kernel, raw_claim_value_kernel, raw_chain_kernel
//                      16-bit caches, raw: the same over the pages of a sequence, the row sums
//                      accumulated in the cache dtype chunk by chunk as the reference does.
//   red_softmax_kernel claim corrections of the raw variant and the softmax of both.
#include "common.h"
#include <type_traits>
#include <math.h>

namespace {

// Sum over the PIECES (16 or 32) consecutive lanes that hold one key row.
template <int PIECES> __device__ __forceinline__ float pieces_sum(float v) {
  static_assert(PIECES == 16 || PIECES == 32, "a key row spans 16 or 32 lanes");
  v = row16_sum(v);
  if (PIECES == 32) v += lane_xor16(v);
  return v;
}
// The valid pages of one block-table row in table order, listed in LDS by the first wave of the
// workgroup (64 entries per step: one load per lane, a ballot ranks the valid ones), instead of a
// serial walk by one thread with a global load per entry.  vpage[n] / vidx[n]: page id / table
// index of the n-th valid page; vord[j]: rank of table entry j or -1; *n_out: their number; *me_out:
// the rank of entry `jp` (0 when it is not valid).  Null pointers are skipped; the caller meets at
// a barrier before reading.
__device__ __forceinline__ void list_valid_pages(const int32_t* __restrict__ row, int NB, int num_pages,
                                                 int jp, int* vpage, int* vidx, int* vord, int* n_out,
                                                 int* me_out) {
  if (threadIdx.x >= 64) return;
  const int lane = threadIdx.x;
  int n = 0;
  if (lane == 0 && me_out) *me_out = 0;
  for (int j0 = 0; j0 < NB; j0 += 64) {
    const int j = j0 + lane;
    const int c = j < NB ? row[j] : -1;
    const int pid = page_is_pad(c) ? -1 : page_id(c);
    const bool ok = pid >= 0 && pid < num_pages;
    const unsigned long long m = __builtin_amdgcn_ballot_w64(ok);
    const int pos = n + __builtin_popcountll(m & lanemask_lt());
    if (ok) {
      if (vpage) vpage[pos] = pid;
      if (vidx) vidx[pos] = j;
      if (me_out && j == jp) *me_out = pos;
    }
    if (vord && j < NB) vord[j] = ok ? pos : -1;
    n += __builtin_popcountll(m);
  }
  if (lane == 0) *n_out = n;
}

// Over the 32 lanes of a wave half: the entry with the largest column index (and its value).
__device__ __forceinline__ void last_claim_reduce(int& c, float& v) {
#define ZP_CLAIM_STEP(OC, OV)              \
  do {                                     \
    const int oc_ = (OC);                  \
    const float ov_ = (OV);                \
    if (oc_ > c) { c = oc_; v = ov_; }     \
  } while (0)
  ZP_CLAIM_STEP(dpp_row_ror<8>(c), dpp_row_ror<8>(v));
  ZP_CLAIM_STEP(dpp_row_ror<4>(c), dpp_row_ror<4>(v));
  ZP_CLAIM_STEP(dpp_row_ror<2>(c), dpp_row_ror<2>(v));
  ZP_CLAIM_STEP(dpp_row_ror<1>(c), dpp_row_ror<1>(v));
  ZP_CLAIM_STEP(lane_xor16(c), lane_xor16(v));
#undef ZP_CLAIM_STEP
}

// A similarity as 2^-32 fixed point (two's complement in an unsigned 64-bit word) and back: sums of
// such words are exact and independent of the order of the additions.
__device__ __forceinline__ unsigned long long to_fixed32(float v) {
  return (unsigned long long)(long long)(v * 4294967296.f);
}
__device__ __forceinline__ float from_fixed32(unsigned long long w) {
  return (float)(long long)w * (1.f / 4294967296.f);
}

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kDmax = 128;
constexpr int TN = 64;                  // keys per column tile
constexpr int ROWF = kDmax + 4;         // floats per LDS row: 16-byte aligned rows whose 16-byte reads by
                                        // eight consecutive rows fall into eight different bank groups
constexpr int KS = kDmax / 2;           // MFMA k-steps (2 per instruction)
constexpr int kChunk = 16;              // columns the reference's all-pairs kernel takes per step
                                        // (BLOCK_N, raw_redudancy_score.py:176)

typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Unpack;
template <> struct Unpack<F32> {
  static constexpr int N = 4;
  __device__ static __forceinline__ void run(const vec16& v, float* o) {
    o[0] = __uint_as_float(v.x); o[1] = __uint_as_float(v.y);
    o[2] = __uint_as_float(v.z); o[3] = __uint_as_float(v.w);
  }
};
template <> struct Unpack<BF16> {
  static constexpr int N = 8;
  __device__ static __forceinline__ void run(const vec16& v, float* o) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};
template <> struct Unpack<F16> {
  static constexpr int N = 8;
  __device__ static __forceinline__ void run(const vec16& v, float* o) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = f16_bits_to_float((uint16_t)(w[i] & 0xffffu));
      o[2 * i + 1] = f16_bits_to_float((uint16_t)(w[i] >> 16));
    }
  }
};

struct GramArgs {
  const char* k;
  const int32_t* table;
  void* r_out;     // lightning: (rows, NB*BS) row sums in the cache dtype
  float* ws_sum;   // raw: fp32 plain row sums
  int32_t* ws_col; // raw: last column over the threshold (logical index, -1 none)
  float* ws_val;   // raw: its value
  float* ws_chunk; // raw, 16-bit caches: [row][T / 16][kDmax] sums of the normalised keys per chunk
  int B, NB, BS, Hkv, D, num_pages;
  int64_t k_sl, k_sp;
  float threshold, eps;
};

template <typename T, bool RAW, int NW>
__global__ __launch_bounds__(NW * 64) void gram_kernel(GramArgs p) {
  constexpr int kThreads = NW * 64, kWaves = NW;    // shadow the file-wide 4-wave constants
  constexpr int NE = Unpack<T>::N;                  // elements per 16-byte piece
  constexpr int PIECES = kDmax / NE;                // pieces per full key row
  constexpr int ROWS_PER_IT = kThreads / PIECES;
  constexpr int STAGE_IT = TN / ROWS_PER_IT;
  constexpr int NSUB = TN / 32;

  extern __shared__ __align__(16) char smem[];
  float* kbuf0 = (float*)smem;
  float* kbuf1 = kbuf0 + TN * ROWF;
  unsigned long long* l_corr = (unsigned long long*)(kbuf1 + TN * ROWF);   // lightning: [BS] claimed from a row
  float* l_sum = (float*)(l_corr + (RAW ? 0 : p.BS));                     //            [BS] row sums
  float* l_val = l_sum + (RAW ? 0 : p.BS);          //            [BS] claimed values
  int* l_col = (int*)(l_val + (RAW ? 0 : p.BS));    //            [BS] claimed columns
  int* vpage = l_col + (RAW ? 0 : p.BS);            // [NB] valid page ids (raw)
  int* vidx = vpage + p.NB;                         // [NB] their table index

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int jp = blockIdx.x % p.NB;                 // row page (table index)
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t orow = (((int64_t)l * p.B + b) * p.Hkv + h);
  const float epsr = Elem<T>::rnd(p.eps);

  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) {  // pad page: logits -inf (lightning); raw marks it in the epilogue
    if (!RAW)
      for (int s = tid; s < p.BS; s += kThreads)
        Elem<T>::st(p.r_out, orow * Tn + (int64_t)jp * p.BS + s, -INFINITY);
    return;
  }

  __shared__ int ncols_s;
  if (RAW) {
    list_valid_pages(p.table + (int64_t)b * p.NB, p.NB, p.num_pages, jp, vpage, vidx, nullptr, &ncols_s, nullptr);
  } else if (tid == 0) {
    vpage[0] = rpid; vidx[0] = jp; ncols_s = 1;
  }
  for (int i = tid; i < 2 * TN * ROWF; i += kThreads) kbuf0[i] = 0.f;
  __syncthreads();
  const int tiles_per_page = p.BS / TN;
  const int ntiles = ncols_s * tiles_per_page;
  const int dpieces = p.D / NE;
  const int64_t k_row = (int64_t)p.Hkv * p.D * T::bytes;
  const char* kbase = p.k + (l * p.k_sl) * T::bytes + (int64_t)h * p.D * T::bytes;

  const int st_piece = tid % PIECES, st_row0 = tid / PIECES;
  vec16 pre[STAGE_IT];
  auto issue_loads = [&](int tile) {
    const int vp = tile / tiles_per_page, toff = (tile - vp * tiles_per_page) * TN;
    const char* src = kbase + (int64_t)vpage[vp] * p.k_sp * T::bytes + (int64_t)toff * k_row;
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      const int row = st_row0 + i * ROWS_PER_IT;
      pre[i] = vec16{0u, 0u, 0u, 0u};
      if (st_piece < dpieces) pre[i] = *(const vec16*)(src + (int64_t)row * k_row + st_piece * 16);
    }
  };
  // normalise (k / max(rnd(|k|), rnd(eps)) in fp32) on the way into LDS
  auto commit_loads = [&](float* buf) {
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      const int row = st_row0 + i * ROWS_PER_IT;
      float e[NE];
      Unpack<T>::run(pre[i], e);
      float ss = 0.f;
#pragma unroll
      for (int q = 0; q < NE; ++q) ss += e[q] * e[q];
      ss = pieces_sum<PIECES>(ss);
      // one reciprocal per key and a multiplication per element (the hardware square root and
      // reciprocal are each within 1 ulp; a division per element would dominate the staging)
      const float rn = __builtin_amdgcn_rcpf(fmaxf(Elem<T>::rnd(__builtin_amdgcn_sqrtf(ss)), epsr));
      if (st_piece < dpieces) {
        float* d = buf + row * ROWF + st_piece * NE;
#pragma unroll
        for (int q = 0; q < NE; q += 2) *(float2*)(d + q) = make_float2(e[q] * rn, e[q + 1] * rn);
      }
    }
  };

  const int row_blocks = p.BS / 32;
  const int NR = (row_blocks + kWaves - 1) / kWaves;
  for (int rr = 0; rr < NR; ++rr) {
    const int rb = rr * kWaves + wave;
    const bool active = rb < row_blocks;
    // ---- A fragments: this lane's key row, normalised.  The order of the contraction index is
    // free as long as both operands agree: k-step 4j + i of wave half `half` takes element
    // 8j + 4 half + i, so a lane's B operands for four steps are one 16-byte LDS read.
    float afrag[KS];
    {
      const int slot = (active ? rb : 0) * 32 + col;
      const char* src = kbase + (int64_t)rpid * p.k_sp * T::bytes + (int64_t)slot * k_row;
      float ss = 0.f;
#pragma unroll
      for (int pc = 0; pc < PIECES; ++pc) {
        float e[NE];
        vec16 v = vec16{0u, 0u, 0u, 0u};
        if (pc < dpieces) v = *(const vec16*)(src + pc * 16);
        Unpack<T>::run(v, e);
#pragma unroll
        for (int q = 0; q < NE; ++q) ss += e[q] * e[q];
        if constexpr (NE == 4) {
          // piece pc holds elements 4 pc .. 4 pc + 3 = (j, half) = (pc / 2, pc % 2)
          if ((pc & 1) == 0) {
#pragma unroll
            for (int q = 0; q < 4; ++q) afrag[(pc >> 1) * 4 + q] = e[q];
          } else if (half) {
#pragma unroll
            for (int q = 0; q < 4; ++q) afrag[(pc >> 1) * 4 + q] = e[q];
          }
        } else {
#pragma unroll
          for (int q = 0; q < NE / 2; ++q) afrag[pc * (NE / 2) + q] = half ? e[2 * q + 1] : e[2 * q];
        }
      }
      const float rn = __builtin_amdgcn_rcpf(fmaxf(Elem<T>::rnd(__builtin_amdgcn_sqrtf(ss)), epsr));
#pragma unroll
      for (int s = 0; s < KS; ++s) afrag[s] = active ? afrag[s] * rn : 0.f;
    }
    float rsum[16], cval[16];
    int ccol[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { rsum[r] = 0.f; cval[r] = 0.f; ccol[r] = -1; }

    if (ntiles > 0) { issue_loads(0); commit_loads(kbuf0); }
    __syncthreads();
    for (int tile = 0; tile < ntiles; ++tile) {
      float* cur = (tile & 1) ? kbuf1 : kbuf0;
      float* nxt = (tile & 1) ? kbuf0 : kbuf1;
      if (tile + 1 < ntiles) issue_loads(tile + 1);
      const int vp = tile / tiles_per_page, toff = (tile - vp * tiles_per_page) * TN;
      const int jc = vidx[vp];
      if (active) {
#pragma unroll
        for (int st = 0; st < NSUB; ++st) {
          f32x16_t acc;
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = 0.f;
          if constexpr (NE == 4) {
            const float4* b4 = (const float4*)(cur + (st * 32 + col) * ROWF + 4 * half);
#pragma unroll
            for (int j4 = 0; j4 < KS / 4; ++j4) {
              const float4 bv = b4[2 * j4];
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * j4 + 0], bv.x, acc, 0, 0, 0);
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * j4 + 1], bv.y, acc, 0, 0, 0);
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * j4 + 2], bv.z, acc, 0, 0, 0);
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * j4 + 3], bv.w, acc, 0, 0, 0);
            }
          } else {
            const float* brow = cur + (st * 32 + col) * ROWF + half;
#pragma unroll
            for (int s = 0; s < KS; ++s)
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[s], brow[2 * s], acc, 0, 0, 0);
          }
          const int cslot = toff + st * 32 + col;
          const int cidx = jc * p.BS + cslot;  // logical column index of this lane
          const bool same_page = jc == jp;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int rslot = rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            float s = acc[r];
            if (same_page && rslot == cslot) s = 0.f;
            rsum[r] += s;
            if (s > p.threshold) { ccol[r] = cidx; cval[r] = s; }
          }
        }
      }
      if (tile + 1 < ntiles) commit_loads(nxt);
      __syncthreads();
    }
    // ---- combine over the 32 lanes of each half (they share rows)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float s = rsum[r];
      int c = ccol[r];
      float v = cval[r];
      s = half_sum(s);
      last_claim_reduce(c, v);
      if (active && col == 0) {
        const int rslot = rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
        if (RAW) {
          const int64_t oi = orow * Tn + (int64_t)jp * p.BS + rslot;
          p.ws_sum[oi] = s;
          p.ws_col[oi] = c;
          p.ws_val[oi] = v;
        } else {
          l_sum[rslot] = s;
          l_col[rslot] = c - jp * p.BS;  // column slot inside the page (or negative)
          l_val[rslot] = v;
        }
      }
    }
  }
  if (!RAW) {
    // every key hands the value of its claimed entry to the row it was taken from; several keys
    // may claim from one row, so the values are added as 2^-32 fixed point: exact to 2^-33 per
    // term and independent of the order (a scan of all keys per row cost ~10 % of the kernel)
    for (int i = tid; i < p.BS; i += kThreads) l_corr[i] = 0ull;
    __syncthreads();
    for (int j = tid; j < p.BS; j += kThreads) {
      const int c = l_col[j];
      if (c >= 0 && c < p.BS) atomicAdd(&l_corr[c], to_fixed32(l_val[j]));
    }
    __syncthreads();
    for (int i = tid; i < p.BS; i += kThreads)
      Elem<T>::st(p.r_out, orow * Tn + (int64_t)jp * p.BS + i, l_sum[i] - from_fixed32(l_corr[i]));
  }
}

// ------------------------------------------------------------------ fp32 products on the fp16 matrix cores
// A normalised key element x (|x| <= 1) is scaled by 2^12 and written as two fp16 numbers,
// h1 = fp16(x') and h2 = fp16(x' - h1), both rounded to nearest: x' - h1 is exact in fp32 (13
// bits), so |x' - h1 - h2| <= 2^-24 |x'|, what rounding a real number to fp32 loses; the scale
// keeps h2 out of fp16's subnormal range for every element that matters (|x| >= 2^-14) and the
// largest scaled element (4096) far below fp16's maximum.  The products h1.g1, h1.g2, h2.g1 are
// exact in the fp32 accumulator, h2.g2 (<= 2^-24 |x||y|) is left out, and the 2^24 of the two
// scales comes off the result exactly.  Three v_mfma_f32_32x32x16_f16 (8 passes each, 16 k) replace eight
// v_mfma_f32_32x32x2_f32 (16 passes each): 3/16 of the matrix-core time at fp32-grade accuracy, and the
// two planes take the LDS bytes of the fp32 element they replace.
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
constexpr float kPlaneScale = 4096.f;                 // 2^12 per operand
constexpr float kPlaneUnscale = 1.f / (4096.f * 4096.f);
constexpr int KSH = kDmax / 16;                       // k-steps of the 16-bit instructions over a key row
constexpr int kPlaneBytes = kDmax * 2;                // one plane of one LDS row; the row keeps ROWF * 4 bytes
__device__ __forceinline__ void split_planes(const float4 e, f16x4_t& h1, f16x4_t& h2) {
  const f32x2_t a = {e.x, e.y}, b = {e.z, e.w};
  const f16x2_t a1 = __builtin_convertvector(a, f16x2_t), b1 = __builtin_convertvector(b, f16x2_t);
  const f32x2_t ar = {e.x - (float)a1[0], e.y - (float)a1[1]}, br = {e.z - (float)b1[0], e.w - (float)b1[1]};
  const f16x2_t a2 = __builtin_convertvector(ar, f16x2_t), b2 = __builtin_convertvector(br, f16x2_t);
  h1 = f16x4_t{a1[0], a1[1], b1[0], b1[1]};
  h2 = f16x4_t{a2[0], a2[1], b2[0], b2[1]};
}
__device__ __forceinline__ f32x16_t mma_planes(const f16x8_t a1, const f16x8_t a2, const f16x8_t b1,
                                               const f16x8_t b2, f32x16_t acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b1, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b2, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b1, acc, 0, 0, 0);
  return acc;
}
// largest of a lane's sixteen tile entries (claims are rare: one maximum per lane and a ballot
// decide whether a tile has any entry over the threshold)
__device__ __forceinline__ float tile_lane_max(const f32x16_t& acc) {
  float m[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
    m[q] = __builtin_fmaxf(__builtin_fmaxf(acc[4 * q], acc[4 * q + 1]), __builtin_fmaxf(acc[4 * q + 2], acc[4 * q + 3]));
  return __builtin_fmaxf(__builtin_fmaxf(m[0], m[1]), __builtin_fmaxf(m[2], m[3]));
}

// ------------------------------------------------------------------ fp32 caches, raw, every pair of pages once
// One workgroup per (layer, sequence, head, valid page a), pages of at most 256 keys.  The
// similarity matrix of a sequence is symmetric, so page a multiplies its rows only with the pages
// (a + d) mod n, d = 0 .. n/2 (the pairs at distance n/2 go to the lower half of the pages when n
// is even).  A tile off the diagonal page serves both of its sides: the rows get their partial
// row sums and their claim (last column over the threshold) as in gram_kernel; the columns get
// the tile's column sums -- slot [d][key], written by exactly one workgroup and added in a fixed
// order by the softmax kernel -- and the last ROW over the threshold as their claim.  Claims meet
// in one 64-bit word per key, (index + 1) << 32 | value bits, through atomicMax: the largest
// index wins whatever the order of the workgroups.
constexpr int kSymWaves = 8;
constexpr int kSymMaxDist = 8;      // column-sum slots per key the workspace holds: tables of <= 16 pages

__global__ void fill_u64_kernel(unsigned long long* dst, int64_t n, unsigned long long v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = v;
}

__global__ __launch_bounds__(kSymWaves * 64) void gram_raw_sym_f32_kernel(GramArgs p) {
  typedef F32 T;
  constexpr int kThreads = kSymWaves * 64;
  constexpr int PIECES = kDmax / 4;                 // 16-byte pieces per key row
  constexpr int ROWS_PER_IT = kThreads / PIECES;    // 16
  constexpr int STAGE_IT = TN / ROWS_PER_IT;        // 4
  constexpr int NSUB = TN / 32;

  extern __shared__ __align__(16) char smem[];
  float* kbuf0 = (float*)smem;
  float* kbuf1 = kbuf0 + TN * ROWF;
  float* l_cpart = kbuf1 + TN * ROWF;               // [2][kSymWaves][TN] column sums per wave and tile
  int* vpage = (int*)(l_cpart + 2 * kSymWaves * TN);
  int* vidx = vpage + p.NB;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int jp = blockIdx.x % p.NB;
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t obase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn;
  unsigned long long* ws_claim = (unsigned long long*)p.ws_col;   // (rows, Tn) words of 64 bits
  const int64_t n_keys = (int64_t)gridDim.x * p.BS;               // == L * B * Hkv * Tn

  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) return;

  __shared__ int nvalid_s, mine_s;
  list_valid_pages(p.table + (int64_t)b * p.NB, p.NB, p.num_pages, jp, vpage, vidx, nullptr, &nvalid_s, &mine_s);
  for (int i = tid; i < 2 * TN * ROWF; i += kThreads) kbuf0[i] = 0.f;
  __syncthreads();
  const int n = nvalid_s, ai = mine_s;
  const int nd = n / 2 + (((n & 1) || ai < n / 2) ? 1 : 0);     // distances 0 .. nd-1
  const int tiles_per_page = p.BS / TN;
  const int ntiles = nd * tiles_per_page;
  // tile / tiles_per_page without a division per tile (at most a few hundred tiles, a handful per page)
  const int tpp_rcp = (65536 + tiles_per_page - 1) / tiles_per_page;
  const int dpieces = p.D / 4;
  const int64_t k_row = (int64_t)p.Hkv * p.D * 4;
  const char* kbase = p.k + (l * p.k_sl) * 4 + (int64_t)h * p.D * 4;

  const int st_piece = tid % PIECES, st_row0 = tid / PIECES;
  vec16 pre[STAGE_IT];
  auto col_page = [&](int d) { return ai + d < n ? ai + d : ai + d - n; };
  auto issue_loads = [&](int tile) {
    const int d = (tile * tpp_rcp) >> 16, toff = (tile - d * tiles_per_page) * TN;
    const char* src = kbase + (int64_t)vpage[col_page(d)] * p.k_sp * 4 + (int64_t)toff * k_row;
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      const int row = st_row0 + i * ROWS_PER_IT;
      pre[i] = vec16{0u, 0u, 0u, 0u};
      if (st_piece < dpieces) pre[i] = *(const vec16*)(src + (int64_t)row * k_row + st_piece * 16);
    }
  };
  auto commit_loads = [&](float* buf) {
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      const int row = st_row0 + i * ROWS_PER_IT;
      float e[4];
      Unpack<T>::run(pre[i], e);
      float ss = (e[0] * e[0] + e[1] * e[1]) + (e[2] * e[2] + e[3] * e[3]);
      ss = pieces_sum<PIECES>(ss);
      const float rn = __builtin_amdgcn_rcpf(fmaxf(__builtin_amdgcn_sqrtf(ss), p.eps)) * kPlaneScale;
      if (st_piece < dpieces) {
        f16x4_t h1, h2;
        split_planes(make_float4(e[0] * rn, e[1] * rn, e[2] * rn, e[3] * rn), h1, h2);
        char* dst = (char*)(buf + row * ROWF) + st_piece * 8;
        *(f16x4_t*)dst = h1;
        *(f16x4_t*)(dst + kPlaneBytes) = h2;
      }
    }
  };

  const int row_blocks = p.BS / 32;
  const int rb = wave;
  const bool active = rb < row_blocks;
  // A fragments: this lane's key row of page a, normalised and split; k-step s of wave half
  // `half` takes elements 16 s + 8 half .. + 7 (pieces 4 s + 2 half and the next one), the same
  // order as the B operand's 16-byte LDS reads
  f16x8_t a1[KSH], a2[KSH];
  {
    const int slot = (active ? rb : 0) * 32 + col;
    const char* src = kbase + (int64_t)rpid * p.k_sp * 4 + (int64_t)slot * k_row;
    float4 mine[2 * KSH];
    float ss = 0.f;
#pragma unroll
    for (int pc = 0; pc < PIECES; ++pc) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (pc < dpieces) v = *(const float4*)(src + pc * 16);
      ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
      if (((pc >> 1) & 1) == 0) mine[(pc >> 2) * 2 + (pc & 1)] = v;
      else if (half) mine[(pc >> 2) * 2 + (pc & 1)] = v;
    }
    const float rn = active ? __builtin_amdgcn_rcpf(fmaxf(__builtin_amdgcn_sqrtf(ss), p.eps)) * kPlaneScale : 0.f;
#pragma unroll
    for (int s = 0; s < KSH; ++s) {
      f16x4_t l1, l2, u1, u2;
      const float4 lo = mine[2 * s], up = mine[2 * s + 1];
      split_planes(make_float4(lo.x * rn, lo.y * rn, lo.z * rn, lo.w * rn), l1, l2);
      split_planes(make_float4(up.x * rn, up.y * rn, up.z * rn, up.w * rn), u1, u2);
      a1[s] = f16x8_t{l1[0], l1[1], l1[2], l1[3], u1[0], u1[1], u1[2], u1[3]};
      a2[s] = f16x8_t{l2[0], l2[1], l2[2], l2[3], u2[0], u2[1], u2[2], u2[3]};
    }
  }
  float rsum[16], cval[16];
  int ccol[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) { rsum[r] = 0.f; cval[r] = 0.f; ccol[r] = -1; }
  const float thr_s = p.threshold * (kPlaneScale * kPlaneScale);
  bool wave_claims = false;       // any tile of this wave with an entry over the threshold (uniform)

  // the column sums of tile t are complete after the barrier that ends it: the waves' shares are
  // added in wave order and stored while tile t+1 is being multiplied
  auto finish_columns = [&](int tile) {
    const int d = (tile * tpp_rcp) >> 16, toff = (tile - d * tiles_per_page) * TN;
    if (d == 0 || tid >= TN) return;
    const float* pt = l_cpart + (tile & 1) * kSymWaves * TN;
    float v = pt[tid];
#pragma unroll
    for (int w2 = 1; w2 < kSymWaves; ++w2) v += pt[w2 * TN + tid];
    const int jc = vidx[col_page(d)];
    p.ws_chunk[(int64_t)(d - 1) * n_keys + obase + (int64_t)jc * p.BS + toff + tid] = v * kPlaneUnscale;
  };

  if (ntiles > 0) { issue_loads(0); commit_loads(kbuf0); }
  __syncthreads();
  for (int tile = 0; tile < ntiles; ++tile) {
    float* cur = (tile & 1) ? kbuf1 : kbuf0;
    float* nxt = (tile & 1) ? kbuf0 : kbuf1;
    if (tile + 1 < ntiles) issue_loads(tile + 1);
    const int d = (tile * tpp_rcp) >> 16, toff = (tile - d * tiles_per_page) * TN;
    const int jc = vidx[col_page(d)];
    float* cpart = l_cpart + ((tile & 1) * kSymWaves + wave) * TN;
#pragma unroll
    for (int st = 0; st < NSUB; ++st) {
      float csum = 0.f, rv = 0.f;
      int rlast = -1;
      if (active) {
        f32x16_t acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        const char* br = (const char*)(cur + (st * 32 + col) * ROWF) + 16 * half;
#pragma unroll
        for (int s = 0; s < KSH; ++s)
          acc = mma_planes(a1[s], a2[s], *(const f16x8_t*)(br + 32 * s),
                           *(const f16x8_t*)(br + kPlaneBytes + 32 * s), acc);
        // sums, claim values and the threshold stay in the planes' scale (a power of two: the
        // same bits come out when it is taken off at the end)
        const int cslot = toff + st * 32 + col;
        const int cidx = jc * p.BS + cslot;   // logical index of this lane's column key
        if (d == 0) {     // the page against itself: a key is not its own neighbour
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3) == cslot) acc[r] = 0.f;
        }
        const bool any_over = __builtin_amdgcn_ballot_w64(tile_lane_max(acc) > thr_s) != 0ull;
        wave_claims |= any_over;
        if (!any_over) {
#pragma unroll
          for (int r = 0; r < 16; ++r) { rsum[r] += acc[r]; csum += acc[r]; }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int rslot = rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            const float sv = acc[r];
            rsum[r] += sv;
            csum += sv;
            const bool over = sv > thr_s;
            if (over && cidx > ccol[r]) { ccol[r] = cidx; cval[r] = sv; }
            if (over) { rlast = rslot; rv = sv; }   // rslot grows with r inside a lane
          }
          if (d != 0) {
            const int orl = lane_xor32(rlast);
            const float orv = lane_xor32(rv);
            if (orl > rlast) { rlast = orl; rv = orv; }
            if (half == 0 && rlast >= 0)   // the column key's claim candidate among page a's rows
              atomicMax(&ws_claim[obase + cidx], ((unsigned long long)(unsigned)(jp * p.BS + rlast + 1) << 32) |
                                                     __float_as_uint(rv * kPlaneUnscale));
          }
        }
      }
      if (d != 0) {
        csum += lane_xor32(csum);
        if (half == 0) cpart[st * 32 + col] = csum;
      }
    }
    if (tile + 1 < ntiles) commit_loads(nxt);
    __syncthreads();
    finish_columns(tile);
  }
  // ---- row side: sums and claims over the 32 lanes of each half
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float sv = half_sum(rsum[r]);
    int c = ccol[r];
    float v = cval[r];
    if (wave_claims) last_claim_reduce(c, v);
    if (active && col == 0) {
      const int64_t oi = obase + (int64_t)jp * p.BS + rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
      p.ws_sum[oi] = sv * kPlaneUnscale;
      if (c >= 0)
        atomicMax(&ws_claim[oi], ((unsigned long long)(unsigned)(c + 1) << 32) | __float_as_uint(v * kPlaneUnscale));
    }
  }
}

// ------------------------------------------------------------------ fp32 caches, lightning, whole page in LDS
// Pages of at most 256 keys; one workgroup per (layer, sequence, head) row walks the row's pages:
// a page is loaded once with coalesced 16-byte loads into registers (requested under the tiles of
// the page before), normalised on the way into LDS (132 KB), and after ONE barrier every wave
// multiplies its 32 rows (A operand read from the same LDS copy) with its share of the column
// blocks (every unordered pair of blocks once): no tile pipeline, no strided row loads.
constexpr int kPage32Rows = 256;
constexpr int kPage32Threads = 512;
__global__ __launch_bounds__(kPage32Threads) void gram_page_f32_kernel(GramArgs p) {
  typedef F32 T;
  constexpr int PIECES = kDmax / 4;                            // 16-byte pieces per key row (32)
  constexpr int ROWS_PER_IT = kPage32Threads / PIECES;         // 16
  constexpr int ITERS = kPage32Rows / ROWS_PER_IT;             // 16
  extern __shared__ __align__(16) char smem[];
  float* kpl = (float*)smem;                                   // [256][ROWF] normalised keys
  unsigned long long* l_corr = (unsigned long long*)(kpl + kPage32Rows * ROWF);
  unsigned long long* l_claim = l_corr + kPage32Rows;       // (claimed index + 1) << 32 | value bits
  float* l_sum = (float*)(l_claim + kPage32Rows);
  float* l_csum = l_sum + kPage32Rows;                        // [4][256] column sums per distance
  int* l_code = (int*)(l_csum + 4 * kPage32Rows);             // [NB] the block table row

  const int tid0 = threadIdx.x;
  // a workgroup walks the pages of one (layer, sequence, kv head) row: the next page's keys are
  // requested into registers under the tiles of this one (a page fills the LDS a CU has, so
  // nothing else could overlap its load)
  const int h = blockIdx.x % p.Hkv;
  const int b = (blockIdx.x / p.Hkv) % p.B;
  const int l = blockIdx.x / (p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t rowbase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn;
  const int dpieces = p.D / 4;
  const int64_t k_row = (int64_t)p.Hkv * p.D * 4;
  const char* layer = p.k + l * p.k_sl * 4 + (int64_t)h * p.D * 4;

  for (int j = tid0; j < p.NB; j += kPage32Threads) l_code[j] = p.table[(int64_t)b * p.NB + j];
  __syncthreads();
  auto page_of = [&](int j) {     // page id of table entry j, or -1 (uniform)
    const int code = __builtin_amdgcn_readfirstlane(l_code[j]);
    const int pid = page_is_pad(code) ? -1 : page_id(code);
    return pid < p.num_pages ? pid : -1;
  };
  auto next_valid = [&](int j) {
    while (j < p.NB && page_of(j) < 0) ++j;
    return j;
  };
  for (int j = 0; j < p.NB; ++j) {      // entries without a page score -inf
    if (page_of(j) >= 0) continue;
    for (int s = tid0; s < p.BS; s += kPage32Threads) Elem<T>::st(p.r_out, rowbase + (int64_t)j * p.BS + s, -INFINITY);
  }
  float4 raw[ITERS];
  auto request = [&](int j, int piece, int prow0) {
    const char* page = layer + (int64_t)page_of(j) * p.k_sp * 4;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int row = it * ROWS_PER_IT + prow0;
      raw[it] = *(const float4*)(page + (int64_t)(row < p.BS ? row : 0) * k_row +
                                 (piece < dpieces ? piece : 0) * 16);
    }
  };
  int jp = next_valid(0);
  if (jp < p.NB) request(jp, tid0 % PIECES, tid0 / PIECES);
#pragma unroll 1
  while (jp < p.NB) {
  // The thread id is made opaque once per page: what is derived from it (LDS addresses, row
  // indices) is then computed where a page uses it, not before the loop and held in registers
  // through all of it, where the prefetched page needs them.
  int tid = tid0;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, col = lane & 31;
  const int piece = tid % PIECES, prow0 = tid / PIECES;
  const int64_t obase = rowbase + (int64_t)jp * p.BS;
  // ---- stage: norms and the normalised copy of the page requested a page ago
  {
    const int row0 = prow0;
    if (tid < kPage32Rows) { l_corr[tid] = 0ull; l_claim[tid] = 0ull; }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int row = it * ROWS_PER_IT + row0;
      if (!(row < p.BS && piece < dpieces)) raw[it] = make_float4(0.f, 0.f, 0.f, 0.f);
      const float4 e = raw[it];
      float ss = (e.x * e.x + e.y * e.y) + (e.z * e.z + e.w * e.w);
      ss = pieces_sum<PIECES>(ss);
      const float rn = __builtin_amdgcn_rcpf(fmaxf(__builtin_amdgcn_sqrtf(ss), p.eps)) * kPlaneScale;
      f16x4_t h1, h2;
      split_planes(make_float4(e.x * rn, e.y * rn, e.z * rn, e.w * rn), h1, h2);
      char* dst = (char*)(kpl + row * ROWF) + piece * 8;
      *(f16x4_t*)dst = h1;
      *(f16x4_t*)(dst + kPlaneBytes) = h2;
    }
  }
  __syncthreads();
  const int nj = next_valid(jp + 1);
  if (nj < p.NB) request(nj, piece, prow0);

  // ---- Gram tiles, every unordered pair of 32-key blocks once: wave a multiplies its block with
  // the blocks (a + d) mod n, d = 0 .. n/2 (the last distance only for the lower half of the
  // waves when n is even).  A tile off the diagonal block serves both of its sides: the rows get
  // their partial row sums and claims as before, the columns get the tile's column sums
  // (slot [d][key], written by exactly one wave, added in a fixed order at the end) and the last
  // ROW over the threshold as their claim.  Claims travel as (index, value) pairs through one
  // 64-bit atomicMax per key, so the result does not depend on the order of the waves.
  const int nrb = p.BS / 32;
  if (wave < nrb) {
    const int rb = wave;
    // lane (col, half) holds elements 16 s + 8 half .. + 7 of key rb * 32 + col for k-step s
    f16x8_t a1[KSH], a2[KSH];
    {
      const char* ar = (const char*)(kpl + (rb * 32 + col) * ROWF) + 16 * half;
#pragma unroll
      for (int s = 0; s < KSH; ++s) {
        a1[s] = *(const f16x8_t*)(ar + 32 * s);
        a2[s] = *(const f16x8_t*)(ar + kPlaneBytes + 32 * s);
      }
    }
    float rsum[16], cval[16];
    int ccol[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { rsum[r] = 0.f; cval[r] = 0.f; ccol[r] = -1; }
    const int nd = nrb / 2 + (((nrb & 1) || rb < nrb / 2) ? 1 : 0);   // distances 0 .. nd-1
    const float thr_s = p.threshold * (kPlaneScale * kPlaneScale);
    bool wave_claims = false;     // any tile of this wave with an entry over the threshold (uniform)
#pragma unroll 1
    for (int d = 0; d < nd; ++d) {
      const int cb = rb + d < nrb ? rb + d : rb + d - nrb;
      f32x16_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
      const char* br = (const char*)(kpl + (cb * 32 + col) * ROWF) + 16 * half;
#pragma unroll
      for (int s = 0; s < KSH; ++s)
        acc = mma_planes(a1[s], a2[s], *(const f16x8_t*)(br + 32 * s),
                         *(const f16x8_t*)(br + kPlaneBytes + 32 * s), acc);
      // sums, claim values and the threshold stay in the planes' scale (a power of two: the same
      // bits come out when it is taken off at the end)
      const int cslot = cb * 32 + col;
      if (d == 0) {     // the block against itself: a key is not its own neighbour
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3) == cslot) acc[r] = 0.f;
      }
      const bool any_over = __builtin_amdgcn_ballot_w64(tile_lane_max(acc) > thr_s) != 0ull;
      wave_claims |= any_over;
      float csum = 0.f, rv = 0.f;     // column side: sum over this lane's rows, last row over the threshold
      int rlast = -1;
      if (!any_over) {
#pragma unroll
        for (int r = 0; r < 16; ++r) { rsum[r] += acc[r]; csum += acc[r]; }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int rslot = rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
          const float sv = acc[r];
          rsum[r] += sv;
          csum += sv;
          const bool over = sv > thr_s;
          if (over && cslot > ccol[r]) { ccol[r] = cslot; cval[r] = sv; }
          if (over) { rlast = rslot; rv = sv; }     // rslot grows with r inside a lane
        }
      }
      if (d != 0) {
        csum += lane_xor32(csum);
        if (half == 0) l_csum[(d - 1) * kPage32Rows + cslot] = csum * kPlaneUnscale;
        if (any_over) {
          const int orl = lane_xor32(rlast);
          const float orv = lane_xor32(rv);
          if (orl > rlast) { rlast = orl; rv = orv; }
          if (half == 0 && rlast >= 0)
            atomicMax(&l_claim[cslot], ((unsigned long long)(unsigned)(rlast + 1) << 32) |
                                           __float_as_uint(rv * kPlaneUnscale));
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float sv = half_sum(rsum[r]);
      int c = ccol[r];
      float v = cval[r];
      if (wave_claims) last_claim_reduce(c, v);
      if (col == 0) {
        const int rslot = rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
        l_sum[rslot] = sv * kPlaneUnscale;
        if (c >= 0)
          atomicMax(&l_claim[rslot], ((unsigned long long)(unsigned)(c + 1) << 32) |
                                         __float_as_uint(v * kPlaneUnscale));
      }
    }
  }
  __syncthreads();
  for (int j = tid; j < p.BS; j += kPage32Threads) {
    const unsigned long long cl = l_claim[j];
    const int c = (int)(cl >> 32) - 1;
    if (c >= 0 && c < p.BS) atomicAdd(&l_corr[c], to_fixed32(__uint_as_float((unsigned)cl)));
  }
  __syncthreads();
  const int ndist = nrb / 2;     // column-side slots in use: distances 1 .. nrb/2
  for (int i = tid; i < p.BS; i += kPage32Threads) {
    float sv = l_sum[i];
    const int blk = i >> 5;
    for (int d = 1; d <= ndist; ++d) {
      // the wave that wrote slot [d][i] is block (blk - d) mod n; with n even the last distance
      // is only run by the lower half of the waves
      const int a = blk - d >= 0 ? blk - d : blk - d + nrb;
      const bool ran = d < nrb / 2 + (((nrb & 1) || a < nrb / 2) ? 1 : 0);
      if (ran) sv += l_csum[(d - 1) * kPage32Rows + i];
    }
    Elem<T>::st(p.r_out, obase + i, sv - from_fixed32(l_corr[i]));
  }
  __syncthreads();   // the page and the per-key slots in LDS are free for the next page
  jp = nj;
  }
}

// ------------------------------------------------------------------ 16-bit caches: split-bf16 Gram
// Same algorithm with the contraction on the bf16 matrix cores.  The fp32 normalised key
// x = k / n is split into hi = bf16(x) and lo = bf16(x - hi); S = hi.hi + hi.lo + lo.hi drops
// only the lo.lo term (relative 2^-18), i.e. fp32-grade dot products at a third of the bf16
// MFMA rate instead of the 16x slower fp32 MFMA.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
constexpr int ROWH = kDmax * 2 + 16;  // bytes per LDS row of one bf16 plane (16 B pad)

__device__ __forceinline__ void split8(const float* x, bf16x8_t& hi, bf16x8_t& lo) {
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const __bf16 h = (__bf16)x[q];
    hi[q] = h;
    lo[q] = (__bf16)(x[q] - (float)h);
  }
}

// NW waves per workgroup: every wave owns one 32-row block of the row page per round, so with 8
// waves a 256-token page needs a single pass over the column tiles (they are normalised and split
// once instead of twice).
template <typename T, bool RAW, int NW>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void gram_split_kernel(GramArgs p) {
  constexpr int kThreads = NW * 64, kWaves = NW;   // shadow the file-wide 4-wave constants
  static_assert(T::bytes == 2, "split path is for 16-bit caches");
  constexpr int PIECES = kDmax / 8;                 // 16-byte pieces per full key row
  constexpr int ROWS_PER_IT = kThreads / PIECES;    // 16
  constexpr int STAGE_IT = TN / ROWS_PER_IT;        // 4
  constexpr int NSUB = TN / 32;
  constexpr int KSB = kDmax / 16;                   // bf16 MFMA k-steps
  constexpr int PLANE = TN * ROWH;                  // bytes of one plane of one buffer

  extern __shared__ __align__(16) char smem[];
  char* buf0 = smem;                                // [hi plane][lo plane]
  char* buf1 = smem + 2 * PLANE;
  unsigned long long* l_corr = (unsigned long long*)(smem + 4 * PLANE);   // [BS] claimed from a row
  float* l_sum = (float*)(l_corr + (RAW ? 0 : p.BS));
  float* l_val = l_sum + (RAW ? 0 : p.BS);
  int* l_col = (int*)(l_val + (RAW ? 0 : p.BS));
  int* vpage = l_col + (RAW ? 0 : p.BS);
  int* vidx = vpage + p.NB;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int jp = blockIdx.x % p.NB;
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t orow = (((int64_t)l * p.B + b) * p.Hkv + h);
  const float epsr = Elem<T>::rnd(p.eps);

  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) {
    if (!RAW)
      for (int s = tid; s < p.BS; s += kThreads)
        Elem<T>::st(p.r_out, orow * Tn + (int64_t)jp * p.BS + s, -INFINITY);
    return;
  }
  __shared__ int ncols_s;
  if (RAW) {
    list_valid_pages(p.table + (int64_t)b * p.NB, p.NB, p.num_pages, jp, vpage, vidx, nullptr, &ncols_s, nullptr);
  } else if (tid == 0) {
    vpage[0] = rpid; vidx[0] = jp; ncols_s = 1;
  }
  for (int i = tid; i < 4 * PLANE / 4; i += kThreads) ((uint32_t*)smem)[i] = 0u;
  __syncthreads();
  const int tiles_per_page = p.BS / TN;
  const int ntiles = ncols_s * tiles_per_page;
  const int dpieces = p.D / 8;
  const int64_t k_row = (int64_t)p.Hkv * p.D * 2;
  const char* kbase = p.k + (l * p.k_sl) * 2 + (int64_t)h * p.D * 2;

  const int st_piece = tid % PIECES, st_row0 = tid / PIECES;
  vec16 pre[STAGE_IT];
  auto issue_loads = [&](int tile) {
    const int vp = tile / tiles_per_page, toff = (tile - vp * tiles_per_page) * TN;
    const char* src = kbase + (int64_t)vpage[vp] * p.k_sp * 2 + (int64_t)toff * k_row;
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      const int row = st_row0 + i * ROWS_PER_IT;
      const int pc = st_piece < dpieces ? st_piece : 0;  // clamp: unconditional load
      pre[i] = *(const vec16*)(src + (int64_t)row * k_row + pc * 16);
    }
  };
  auto commit_loads = [&](char* buf) {
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      const int row = st_row0 + i * ROWS_PER_IT;
      float e[8];
      Unpack<T>::run(pre[i], e);
      float ss = 0.f;
      if (st_piece < dpieces) {
#pragma unroll
        for (int q = 0; q < 8; ++q) ss += e[q] * e[q];
      }
      ss = pieces_sum<PIECES>(ss);
      const float n = fmaxf(Elem<T>::rnd(sqrtf(ss)), epsr);
      if (st_piece < dpieces) {
#pragma unroll
        for (int q = 0; q < 8; ++q) e[q] = e[q] / n;
        bf16x8_t hi, lo;
        split8(e, hi, lo);
        *(bf16x8_t*)(buf + row * ROWH + st_piece * 16) = hi;
        *(bf16x8_t*)(buf + PLANE + row * ROWH + st_piece * 16) = lo;
      }
    }
  };

  const int row_blocks = p.BS / 32;
  const int NR = (row_blocks + kWaves - 1) / kWaves;
  for (int rr = 0; rr < NR; ++rr) {
    const int rb = rr * kWaves + wave;
    const bool active = rb < row_blocks;
    // ---- A fragments: this lane's key row; lane (row, half) holds k = 16 s + 8 half + i
    bf16x8_t ahi[KSB], alo[KSB];
    {
      const int slot = (active ? rb : 0) * 32 + col;
      const char* src = kbase + (int64_t)rpid * p.k_sp * 2 + (int64_t)slot * k_row;
      float x[KSB][8];
      float ss = 0.f;
#pragma unroll
      for (int s = 0; s < KSB; ++s) {
        const int pc = 2 * s + half;
        vec16 v = vec16{0u, 0u, 0u, 0u};
        if (pc < dpieces) v = *(const vec16*)(src + pc * 16);
        Unpack<T>::run(v, x[s]);
#pragma unroll
        for (int q = 0; q < 8; ++q) ss += x[s][q] * x[s][q];
      }
      ss += lane_xor32(ss);  // the other half of the row
      const float n = fmaxf(Elem<T>::rnd(sqrtf(ss)), epsr);
#pragma unroll
      for (int s = 0; s < KSB; ++s) {
#pragma unroll
        for (int q = 0; q < 8; ++q) x[s][q] = active ? x[s][q] / n : 0.f;
        split8(x[s], ahi[s], alo[s]);
      }
    }
    float rsum[16], cval[16];
    int ccol[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { rsum[r] = 0.f; cval[r] = 0.f; ccol[r] = -1; }

    if (ntiles > 0) { issue_loads(0); commit_loads(buf0); }
    __syncthreads();
    for (int tile = 0; tile < ntiles; ++tile) {
      char* cur = (tile & 1) ? buf1 : buf0;
      char* nxt = (tile & 1) ? buf0 : buf1;
      if (tile + 1 < ntiles) issue_loads(tile + 1);
      const int vp = tile / tiles_per_page, toff = (tile - vp * tiles_per_page) * TN;
      const int jc = vidx[vp];
      if (active) {
#pragma unroll 1
        for (int st = 0; st < NSUB; ++st) {
          f32x16_t acc;
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = 0.f;
          const char* brow = cur + (st * 32 + col) * ROWH + half * 16;
#pragma unroll
          for (int s0 = 0; s0 < KSB; s0 += 4) {
            bf16x8_t bh[4], bl[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              bh[s] = *(const bf16x8_t*)(brow + (s0 + s) * 32);
              bl[s] = *(const bf16x8_t*)(brow + PLANE + (s0 + s) * 32);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[s0 + s], bh[s], acc, 0, 0, 0);
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[s0 + s], bl[s], acc, 0, 0, 0);
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(alo[s0 + s], bh[s], acc, 0, 0, 0);
            }
          }
          const int cslot = toff + st * 32 + col;
          const int cidx = jc * p.BS + cslot;
          const bool same_page = jc == jp;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int rslot = rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            float s = acc[r];
            if (same_page && rslot == cslot) s = 0.f;
            rsum[r] += s;
            if (s > p.threshold) { ccol[r] = cidx; cval[r] = s; }
          }
        }
      }
      if (tile + 1 < ntiles) commit_loads(nxt);
      __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float s = rsum[r];
      int c = ccol[r];
      float v = cval[r];
      s = half_sum(s);
      last_claim_reduce(c, v);
      if (active && col == 0) {
        const int rslot = rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
        if (RAW) {
          const int64_t oi = orow * Tn + (int64_t)jp * p.BS + rslot;
          p.ws_sum[oi] = s;
          p.ws_col[oi] = c;
          p.ws_val[oi] = v;
        } else {
          l_sum[rslot] = s;
          l_col[rslot] = c - jp * p.BS;
          l_val[rslot] = v;
        }
      }
    }
  }
  if (!RAW) {
    // claim values go to the rows they were taken from as 2^-32 fixed-point atomics
    // (order-independent), not through a scan of all claims per row
    for (int i = tid; i < p.BS; i += kThreads) l_corr[i] = 0ull;
    __syncthreads();
    for (int j = tid; j < p.BS; j += kThreads) {
      const int c = l_col[j];
      if (c >= 0 && c < p.BS) atomicAdd(&l_corr[c], to_fixed32(l_val[j]));
    }
    __syncthreads();
    for (int i = tid; i < p.BS; i += kThreads)
      Elem<T>::st(p.r_out, orow * Tn + (int64_t)jp * p.BS + i, l_sum[i] - from_fixed32(l_corr[i]));
  }
}

// ------------------------------------------------------------------ lightning, whole page in LDS
// Per-page variant for 16-bit caches and pages of up to 256 keys: the page is normalised and
// split once into LDS (hi and lo planes, 2 x 68 KB).  The Gram matrix is symmetric, so every
// unordered pair of 32-key blocks is multiplied once: wave a takes the blocks (a, a+d mod n)
// for d = 0..n/2 (the pairs at distance n/2 go to the lower half of the waves), which is 5 or 4
// tiles per wave for a 256-key page instead of 8.  A tile only feeds the claim rule (its
// entries over the threshold update the last-column-over-threshold of the keys on BOTH of its
// sides); the row sums do not need the matrix at all:
//     sum_{j != i} e_i.e_j = e_i . (sum_j e_j - e_i)
// is one fp32 dot product per key against the page's summed key, done while the raw keys are
// still in registers.  The values of the (at most one per key) claimed entries are recomputed
// afterwards from the two planes.
constexpr int kPageThreads = 512;
constexpr int kPageWaves = kPageThreads / 64;
constexpr int kPageRows = 256;

// Two floats to packed bf16 (round to nearest even) in one v_cvt_pk_bf16_f32.
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_bf16(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, bf16x2_t));
}
// hi = bf16(x), lo = bf16(x - hi) for eight values, packed pairwise.
__device__ __forceinline__ void split8_pk(const float* x, u32x4& hi, u32x4& lo) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t h = pk_bf16(x[2 * i], x[2 * i + 1]);
    hi[i] = h;
    lo[i] = pk_bf16(x[2 * i] - __uint_as_float(h << 16), x[2 * i + 1] - __uint_as_float(h & 0xffff0000u));
  }
}


// Largest value over the 32 lanes of a wave half.
__device__ __forceinline__ int half_max_i(int v) {
  v = max(v, dpp_row_ror<8>(v));
  v = max(v, dpp_row_ror<4>(v));
  v = max(v, dpp_row_ror<2>(v));
  v = max(v, dpp_row_ror<1>(v));
  return max(v, lane_xor16(v));
}

// The 16-bit MFMA of the cache dtype: products of cache elements are exact in fp32.
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
template <typename T> struct Mfma16;
template <> struct Mfma16<BF16> {
  typedef bf16x8_t V;
  __device__ static __forceinline__ f32x16_t run(V a, V b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<F16> {
  typedef f16x8_t V;
  __device__ static __forceinline__ f32x16_t run(V a, V b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// A float as three 16-bit pieces of the cache dtype (hi + mid + lo carries its fp32 mantissa).
template <typename T> struct Split3;
template <> struct Split3<BF16> {
  __device__ static __forceinline__ void run(float v, uint16_t* o) {
    const float h = bf16_round(v), m = bf16_round(v - h), l = bf16_round(v - h - m);
    o[0] = (uint16_t)(__float_as_uint(h) >> 16);
    o[1] = (uint16_t)(__float_as_uint(m) >> 16);
    o[2] = (uint16_t)(__float_as_uint(l) >> 16);
  }
};
template <> struct Split3<F16> {
  __device__ static __forceinline__ void run(float v, uint16_t* o) {
    o[0] = float_to_f16_bits(v);
    const float r1 = v - f16_bits_to_float(o[0]);
    o[1] = float_to_f16_bits(r1);
    o[2] = float_to_f16_bits(r1 - f16_bits_to_float(o[1]));
  }
};

// The cosine matrix factors as S_ij = rn_i rn_j (k_i . k_j) with rn = 1 / norm: the raw 16-bit
// keys go to the matrix cores as they are (one MFMA per k-step, exact products, fp32 sums) and
// the two scale factors are applied to the accumulators.  Sixteen waves share a compute unit's
// four vector units, and vector instruction issue is the first thing they run out of, so
// everything that can be is kept off the vector ALUs:
//   * the page goes from global memory straight into LDS (no staging registers, no LDS stores);
//     a load instruction moves four key rows, which sit 1040 bytes apart in groups of four so that
//     the matrix cores' fragment reads spread over the banks: piece g (16 bytes) of row r of a
//     group at (g / 4) * 256 + r * 64 + (g % 4) * 16;
//   * wave a loads row block a, so it can take the block's norms from the diagonal of its own
//     Gram tile (which the claim rule needs anyway) before any barrier;
//   * the summed normalised key  sum_j rn_j k_j  is a matrix product too, contracted over the
//     keys: A = rn as three 16-bit pieces (rows 0..2), B = the keys read through the transposing
//     LDS load (`ds_read_b64_tr_b16`: lane i of sixteen receives column i of a 4 x 16 block).
// One plane of raw keys in LDS (65 KB), so two workgroups share a compute unit.  A workgroup
// walks the pages of one row: once the tiles of a page are done nothing reads its keys in LDS
// any more, so the next page is requested then and lands while the row sums are finished.
constexpr int kPgGrp = 1040;                          // bytes from one group of four key rows to the next
constexpr int kPgBytes = (kPageRows / 4) * kPgGrp;    // the page in LDS
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef void __attribute__((address_space(3))) * lds_ptr_t;

#ifdef ZP_PAGE_STAMP
// Measurement build: thread 0 of every workgroup records the core-clock counter at the phase
// boundaries and the constant-rate counter at both ends.
constexpr int kPageStampMax = 1 << 16;
__device__ long long zp_page_stamp_buf[kPageStampMax * 12];
extern "C" int zp_debug_page_stamps(long long* dst, int n_groups) {
  return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(zp_page_stamp_buf), (size_t)n_groups * 12 * 8);
}
#define ZP_PSTAMP() do { if (tid == 0 && nst < 10) st_[nst++] = clock64(); } while (0)
#else
#define ZP_PSTAMP() do { } while (0)
#endif

// 1 / norm as 16-bit pieces for the matrix cores.  bf16 has fp32's exponent range: three pieces
// carry all 24 mantissa bits.  fp16 does not: the pieces are taken of rn * 2^-x with x chosen per
// block of 32 keys so that the block's largest value sits at the top of fp16's range, which leaves
// 39 bits below it; the accumulator is rescaled where the block changes.
template <typename T> struct RnScale;
template <> struct RnScale<BF16> { static constexpr bool per_block = false; };
template <> struct RnScale<F16> { static constexpr bool per_block = true; };

template <typename T>
__global__ __launch_bounds__(kPageThreads, 4) void gram_page_kernel(GramArgs p) {
  static_assert(T::bytes == 2, "16-bit caches only");
  typedef typename Mfma16<T>::V frag_t;
  constexpr int PIECES = kDmax / 8;
  constexpr int KSB = kDmax / 16;

  extern __shared__ __align__(16) char smem[];
  char* k_pl = smem;                                   // raw keys
  char* s_pl = smem + kPgBytes;                        // [4][kDmax] 16-bit: summed key as hi, mid, lo; zeros
  char* rn_pl = s_pl + 4 * kDmax * 2;                  // [4][kPageRows] 16-bit: 1 / norm as hi, mid, lo; zeros
  // claimed from a row / row sums: two copies, taken in turn by the pages of the walk, because a
  // page's last phase reads them while the next page's first phase writes them
  unsigned long long* l_corr2 = (unsigned long long*)(rn_pl + 4 * kPageRows * 2);
  float* l_sum2 = (float*)(l_corr2 + 2 * kPageRows);
  float* l_rn = l_sum2 + 2 * kPageRows;                // 1 / norm
  int* l_col = (int*)(l_rn + kPageRows);
  int* l_bexp = l_col + kPageRows;                     // [kPageWaves] scale exponent of a block's rn pieces
  int* l_code = l_bexp + kPageWaves;                   // [NB] the block table row

  const int tid = threadIdx.x;
#ifdef ZP_PAGE_STAMP
  long long st_[10];
  int nst = 0;
#endif
  // a workgroup walks the pages of one (layer, sequence, kv head) row
  const int h = blockIdx.x % p.Hkv;
  const int b = (blockIdx.x / p.Hkv) % p.B;
  const int l = blockIdx.x / (p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t rowbase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn;
  const float epsr = Elem<T>::rnd(p.eps);
  const int dpieces = p.D / 8;
  const int k_row = p.Hkv * p.D * 2;
  const char* layer = p.k + l * p.k_sl * 2 + (int64_t)h * p.D * 2;
  const int nrb = p.BS / 32;

  for (int j = tid; j < p.NB; j += kPageThreads) l_code[j] = p.table[(int64_t)b * p.NB + j];
  if (tid < kDmax / 2) ((uint32_t*)(s_pl + 3 * kDmax * 2))[tid] = 0u;
  else if (tid < kDmax / 2 + kPageRows / 2) ((uint32_t*)(rn_pl + 3 * kPageRows * 2))[tid - kDmax / 2] = 0u;
  if (dpieces < PIECES) {   // the tail of every key row must read as zero
    for (int i = tid; i < kPgBytes / 4; i += kPageThreads) ((uint32_t*)k_pl)[i] = 0u;
  }
  __syncthreads();
  // page id of table entry j, or -1 (wave-uniform)
  auto page_of = [&](int j) {
    const int code = __builtin_amdgcn_readfirstlane(l_code[j]);
    const int pid = page_is_pad(code) ? -1 : page_id(code);
    return pid < p.num_pages ? pid : -1;
  };
  auto next_valid = [&](int j) {
    while (j < p.NB && page_of(j) < 0) ++j;
    return j;
  };
  for (int j = 0; j < p.NB; ++j) {      // entries without a page score -inf
    if (page_of(j) >= 0) continue;
    for (int s = tid; s < p.BS; s += kPageThreads) Elem<T>::st(p.r_out, rowbase + (int64_t)j * p.BS + s, -INFINITY);
  }
  // ---- a page into LDS: wave w requests row block w, eight instructions of four rows
  auto request = [&](int j, int w, int ln) {
    if (w >= nrb) return;
    const int st_g = (ln >> 4) * 4 + (ln & 3), st_r = (ln >> 2) & 3;
    const char* page = layer + (int64_t)page_of(j) * p.k_sp * 2;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(page + (int64_t)w * 32 * k_row), 0, 32 * k_row, 0x00020000);
    const int voff = st_r * k_row + st_g * 16;
    if (st_g < dpieces) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)(k_pl + (w * 8 + i) * kPgGrp), 16, voff,
                                                 i * 4 * k_row, 0, 0);
    }
  };

  int jp = next_valid(0);
  if (jp < p.NB) request(jp, __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
  int par = 0;
#pragma unroll 1
  while (jp < p.NB) {
    // Lane and wave numbers are made opaque once per page: what is derived from them (LDS
    // addresses, row indices) is then computed where a page uses it instead of once before the
    // loop and held in registers through all of it, which the tiles have none to spare for.
    int lane = tid & 63;
    asm volatile("" : "+v"(lane));
    int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    asm volatile("" : "+s"(wave));
    const int half = lane >> 5, col = lane & 31;
    const int a = wave;
    // fragment of k-step s of this lane's row: base + (s / 2) * 256 + (s % 2) * 32
    const int rd_off = (col >> 2) * kPgGrp + (col & 3) * 64 + half * 16;
#ifdef ZP_PAGE_STAMP
    nst = 0;
    const long long wall0 = wall_clock64();
#endif
    ZP_PSTAMP();
    unsigned long long* l_corr = l_corr2 + par * kPageRows;
    float* l_sum = l_sum2 + par * kPageRows;
    const char* page = layer + (int64_t)page_of(jp) * p.k_sp * 2;
    const int64_t obase = rowbase + (int64_t)jp * p.BS;
    const int tix = wave * 64 + lane;
    if (tix < kPageRows) { l_col[tix] = -1; l_corr[tix] = 0ull; }
    ZP_PSTAMP();   // 1

    // ---- norms from the diagonal of the Gram matrix: wave a multiplies its own block (a, a) as
    // soon as its own rows have landed; the 32 lanes that hold a diagonal entry turn it into 1 / norm
    frag_t ak[KSB];
    f32x16_t diag;
#pragma unroll
    for (int r = 0; r < 16; ++r) diag[r] = 0.f;
    if (wave < nrb) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const char* arow = k_pl + a * 8 * kPgGrp + rd_off;
#pragma unroll
      for (int s = 0; s < KSB; ++s) ak[s] = *(const frag_t*)(arow + (s >> 1) * 256 + (s & 1) * 32);
#pragma unroll
      for (int s = 0; s < KSB; ++s) diag = Mfma16<T>::run(ak[s], ak[s], diag);
      // lane (col, half) owns rows (r/4)*8 + half*4 + r%4 of column col: entry (col, col) is its
      // register (col/8)*4 + col%4 when (col%8)/4 == half
      const int my_r = (col >> 3) * 4 + (col & 3);
      float ss = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) ss = r == my_r ? diag[r] : ss;
      const bool mine = ((col & 7) >> 2) == half;
      // the quotient only scales fp32 sums: the 1-ulp reciprocal is exact enough
      const float rn = __builtin_amdgcn_rcpf(fmaxf(Elem<T>::rnd(sqrtf(ss)), epsr));
      float f = rn;
      if constexpr (RnScale<T>::per_block) {
        int e = mine ? (int)((__float_as_uint(rn) >> 23) & 0xffu) : 0;   // biased exponent
        e = half_max_i(e);
        e = max(e, lane_xor32(e));
        const int x = e - 127 - 14;          // rn = f * 2^x, the block's largest f in [2^14, 2^15)
        f = ldexpf(rn, -x);
        if (lane == 0) l_bexp[a] = x;
      }
      if (mine) {
        l_rn[a * 32 + col] = rn;
        l_sum[a * 32 + col] = ss * rn * rn;      // |e_i|^2, taken off the row sum below
        uint16_t o[3];
        Split3<T>::run(f, o);
#pragma unroll
        for (int pl = 0; pl < 3; ++pl) *(uint16_t*)(rn_pl + pl * kPageRows * 2 + (a * 32 + col) * 2) = o[pl];
      }
    }
    ZP_PSTAMP();   // 2: norms of wave 0's block
    __syncthreads();
    ZP_PSTAMP();   // 3: page and norms complete

    // ---- summed normalised key S = sum_j rn_j k_j on the matrix cores, by the upper four waves
    // (which have one tile fewer below): wave 7 - t takes the head dims 32 t .. 32 t + 31 and walks
    // the keys sixteen at a time.  A: rows 0..2 = the pieces of rn (lanes col >= 3 read zeros);
    // B: the keys transposed.  The three rows of the result are added smallest first and stored as
    // three 16-bit planes, so that the matrix cores can multiply the keys with S as well.
    if (wave >= kPageWaves - 4) {
      // these four waves carry the key sum on top of their tiles and are what the barrier behind
      // the tiles waits for: they issue ahead of the other waves of the compute unit until then
      __builtin_amdgcn_s_setprio(2);
      const int dt = kPageWaves - 1 - wave;
      f32x16_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
      const char* asrc = rn_pl + (col < 3 ? col : 3) * kPageRows * 2 + half * 16;
      // transposing read: lane i of a group of sixteen supplies the address of key row i / 4, four
      // dims at (i % 4) * 4 of the group's sixteen dims; groups: (half, dims 16 (g & 1) ..)
      const int i16 = lane & 15, g4 = lane >> 4;
      const char* bsrc = k_pl + (g4 >> 1) * 2 * kPgGrp + dt * 256 + (i16 >> 2) * 64 +
                         ((g4 & 1) * 2 + ((i16 & 3) >> 1)) * 16 + (i16 & 1) * 8;
      // a block of 32 keys is two k-steps; the operands of the next block are requested before the
      // products of this one, so the chain of dependent products does not also wait for LDS
      int xcur = 0;
      frag_t af[2][2];
      s16x4_t bl[2][2], bh[2][2];
      auto fetch = [&](int blk, auto buf) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int ks = 2 * blk + u;
          af[buf.value][u] = *(const frag_t*)(asrc + ks * 32);
          bl[buf.value][u] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4_t __attribute__((address_space(3)))*)(bsrc + ks * 4 * kPgGrp));
          bh[buf.value][u] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4_t __attribute__((address_space(3)))*)(bsrc + (ks * 4 + 1) * kPgGrp));
        }
      };
      auto products = [&](int blk, auto buf) {
        if constexpr (RnScale<T>::per_block) {
          const int xb = l_bexp[blk];
          if (blk > 0) {
#pragma unroll
            for (int r = 0; r < 3; ++r) acc[r] = ldexpf(acc[r], xcur - xb);
          }
          xcur = xb;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const s16x8_t bb = __builtin_shufflevector(bl[buf.value][u], bh[buf.value][u], 0, 1, 2, 3, 4, 5, 6, 7);
          acc = Mfma16<T>::run(af[buf.value][u], __builtin_bit_cast(frag_t, bb), acc);
        }
      };
      typedef std::integral_constant<int, 0> B0;
      typedef std::integral_constant<int, 1> B1;
      fetch(0, B0{});
#pragma unroll 1
      for (int blk = 0; blk < nrb; blk += 2) {
        if (blk + 1 < nrb) fetch(blk + 1, B1{});
        products(blk, B0{});
        if (blk + 1 < nrb) {
          if (blk + 2 < nrb) fetch(blk + 2, B0{});
          products(blk + 1, B1{});
        }
      }
      if (half == 0) {
        float sv = (acc[2] + acc[1]) + acc[0];
        if constexpr (RnScale<T>::per_block) sv = ldexpf(sv, xcur);
        uint16_t o[3];
        Split3<T>::run(sv, o);
#pragma unroll
        for (int pl = 0; pl < 3; ++pl) *(uint16_t*)(s_pl + pl * kDmax * 2 + (dt * 32 + col) * 2) = o[pl];
      }
    }
    ZP_PSTAMP();   // 4: (wave 0 has nothing to do for the key sum)

    // ---- Gram tiles: wave a owns row block a and the column blocks (a + d) mod n
    float rn_row[16];
    if (wave < nrb) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {   // the lane's rows come in runs of four
        const float4 v = *(const float4*)(l_rn + a * 32 + q * 8 + half * 4);
        rn_row[4 * q] = v.x; rn_row[4 * q + 1] = v.y; rn_row[4 * q + 2] = v.z; rn_row[4 * q + 3] = v.w;
      }
      // a tile whose largest entry stays below this cannot hold a claim (slack for the rounding of
      // the two ways the scale factors are multiplied in)
      const float thr_lo = p.threshold - fabsf(p.threshold) * 1e-5f - 1e-30f;
      float rn_max = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) rn_max = fmaxf(rn_max, rn_row[r]);
      int dcol[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) dcol[r] = -1;
      const int nd = nrb / 2 + ((nrb & 1) || a < nrb / 2 ? 1 : 0);   // distances 0 .. nd-1
      // what a tile feeds: the last column over the threshold of the keys on both of its sides
      auto scan = [&](const f32x16_t& acc, int cb, bool off_diagonal) {
        const int cslot = cb * 32 + col;
        const float rn_col = l_rn[cslot];
        // most tiles hold no entry over the threshold, and one maximum decides.  With a positive
        // threshold only positive products matter, and those are at most the largest product
        // times the largest row factor: that bound needs no multiplication per entry.
        if (thr_lo > 0.f) {
          float amax = 0.f;
#pragma unroll
          for (int r = 0; r < 16; ++r) amax = fmaxf(amax, acc[r]);
          if (!__any(amax * rn_max * rn_col > thr_lo)) return;
        }
        float big = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) big = fmaxf(big, acc[r] * rn_row[r]);
        if (!__any(big * rn_col > thr_lo)) return;
        // row side: key (a, r) sees column cslot; column side (off the diagonal block, where both
        // (i, j) and (j, i) are computed): key cslot sees the rows of block a, whose index grows
        // with r inside a lane, so the last hit is the largest
        int rlast = -1;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const bool over = acc[r] * (rn_row[r] * rn_col) > p.threshold;
          dcol[r] = max(dcol[r], over ? cslot : -1);
          rlast = over ? r : rlast;
        }
        if (off_diagonal && __any(rlast >= 0)) {
          int ci = rlast < 0 ? -1 : a * 32 + (rlast >> 2) * 8 + half * 4 + (rlast & 3);
          ci = max(ci, lane_xor32(ci));
          if (half == 0 && ci >= 0) atomicMax(&l_col[cslot], ci);
        }
      };
      {
        // the diagonal block was multiplied for the norms; a key against itself counts as 0
        f32x16_t acc;
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[r] = (r >> 2) * 8 + half * 4 + (r & 3) == col ? 0.f : diag[r];
        scan(acc, a, false);
      }
#pragma unroll 1
      for (int d = 1; d < nd; ++d) {
        const int cb = a + d < nrb ? a + d : a + d - nrb;
        const char* brow = k_pl + cb * 8 * kPgGrp + rd_off;
        f32x16_t acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        frag_t bk[KSB];
#pragma unroll
        for (int s = 0; s < KSB; ++s) bk[s] = *(const frag_t*)(brow + (s >> 1) * 256 + (s & 1) * 32);
#pragma unroll
        for (int s = 0; s < KSB; ++s) acc = Mfma16<T>::run(ak[s], bk[s], acc);
        scan(acc, cb, true);
      }
      // most waves see no entry over the threshold: then the reduction over the lanes is skipped
      bool mine = false;
#pragma unroll
      for (int r = 0; r < 16; ++r) mine |= dcol[r] >= 0;
      if (__any(mine)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int c = half_max_i(dcol[r]);
          if (col == 0 && c >= 0)
            atomicMax(&l_col[a * 32 + (r >> 2) * 8 + half * 4 + (r & 3)], c);
        }
      }
    }
    ZP_PSTAMP();   // 5: tiles of wave 0
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();
    ZP_PSTAMP();   // 6: tiles of all waves, key sum planes

    // ---- nothing below reads the page in LDS: the next page of the row is requested now and
    // lands while this one finishes
    const int nj = next_valid(jp + 1);
    if (nj < p.NB) request(nj, wave, lane);

    // ---- row sums without the matrix: sum_{j != i} e_i.e_j = rn_i (k_i . S) - |e_i|^2, the products
    // k_i . S as one more tile whose columns 0..2 are the planes of S (the other lanes read zeros)
    if (wave < nrb) {
      f32x16_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
      const char* srow = s_pl + (col < 3 ? col : 3) * kDmax * 2 + half * 16;
#pragma unroll
      for (int s = 0; s < KSB; ++s) acc = Mfma16<T>::run(ak[s], *(const frag_t*)(srow + s * 32), acc);
      float t[16];
#pragma unroll
      for (int r = 0; r < 16; ++r)   // lane col 0 adds the lo, mid and hi products (lanes col 2, 1, 0), smallest first
        t[r] = (dpp_row_shl<2>(acc[r]) + dpp_row_shl<1>(acc[r])) + acc[r];
      if (col == 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float4* dst = (float4*)(l_sum + a * 32 + q * 8 + half * 4);
          float4 v = *dst;
          v.x = t[4 * q] * rn_row[4 * q] - v.x;
          v.y = t[4 * q + 1] * rn_row[4 * q + 1] - v.y;
          v.z = t[4 * q + 2] * rn_row[4 * q + 2] - v.z;
          v.w = t[4 * q + 3] * rn_row[4 * q + 3] - v.w;
          *dst = v;
        }
      }
    }
    // ---- value of every key's claimed entry, subtracted from the row it was taken from.  Several
    // keys may claim from one row: the values are added as 2^-32 fixed point with integer atomics,
    // which is exact for a cosine above 2^-8 and does not depend on the order of the additions.
    // Wave w looks at the keys 32 w .. 32 w + 31 at once (most have no claim) and then handles the
    // ones that have, four at a time with sixteen lanes per key; the two key rows come from
    // global memory (the cache: the page was read a moment ago).
    {
      static_assert(PIECES == 16, "sixteen lanes per key");
      const int key = wave * 32 + col;
      const int cl = key < p.BS ? l_col[key] : -1;
      // cl == key: with a negative threshold the zeroed diagonal entry itself can be the claim; its
      // value is 0, nothing to hand back
      unsigned todo = (unsigned)__builtin_amdgcn_ballot_w64(half == 0 && cl >= 0 && cl != key);
      const int q = lane >> 4, piece = lane & 15;
      while (todo) {
        unsigned m = todo;           // the q-th lowest key with a claim goes to lane group q
#pragma unroll
        for (int i = 0; i < 3; ++i) m = i < q ? m & (m - 1) : m;
        const int jl = m ? __builtin_ctz(m) : -1;
#pragma unroll
        for (int i = 0; i < 4; ++i) todo &= todo - 1;
        const int c = __builtin_amdgcn_ds_bpermute((jl < 0 ? 0 : jl) << 2, cl);
        if (jl >= 0) {               // uniform over the 16 lanes of a key
          const int j = wave * 32 + jl;
          u32x4 kj = u32x4{0u, 0u, 0u, 0u}, kc = kj;
          if (piece < dpieces) {
            kj = *(const u32x4*)(page + (int64_t)j * k_row + piece * 16);
            kc = *(const u32x4*)(page + (int64_t)c * k_row + piece * 16);
          }
          float ej[8], ec[8];
          Unpack<T>::run(vec16{kj.x, kj.y, kj.z, kj.w}, ej);
          Unpack<T>::run(vec16{kc.x, kc.y, kc.z, kc.w}, ec);
          float t = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) t = fmaf(ej[e], ec[e], t);
          t = pieces_sum<PIECES>(t);
          if (piece == 0) atomicAdd(&l_corr[c], to_fixed32(t * (l_rn[j] * l_rn[c])));
        }
      }
    }
    ZP_PSTAMP();   // 7: row sums and claim values of wave 0
    __syncthreads();
    ZP_PSTAMP();   // 8
    if (tix < p.BS) Elem<T>::st(p.r_out, obase + tix, l_sum[tix] - from_fixed32(l_corr[tix]));
#ifdef ZP_PAGE_STAMP
    ZP_PSTAMP();   // 9
    if (tid == 0 && blockIdx.x * p.NB + jp < kPageStampMax) {
      long long* dst = zp_page_stamp_buf + ((int64_t)blockIdx.x * p.NB + jp) * 12;
      for (int i = 0; i < 10; ++i) dst[i] = i < nst ? st_[i] : 0;
      dst[10] = wall0;
      dst[11] = wall_clock64() - wall0;
    }
#endif
    jp = nj;
    par ^= 1;
  }
}
#undef ZP_PSTAMP

// ------------------------------------------------------------------ raw, 16-bit caches
// All-pairs variant over the whole sequence.  Four launches; the claims use the symmetric scheme
// of the page kernel above, with pages in the role of its 32-key blocks:
//   1. raw_prep_kernel: 1 / norm of every key, the sum of the normalised keys of every 16-key
//      chunk; claims start at "none".
//   2. gram_raw_kernel: one workgroup per valid page a; it multiplies page a with the pages
//      (a + d) mod n, d = 0..n/2, so every unordered pair of pages is done once, and records for
//      the keys on both sides the last (logical) column over the threshold with integer
//      atomic maxima (order-independent, so the result is deterministic).
//   3. raw_claim_value_kernel: the fp32 value of every key's claimed entry.
//   4. raw_chain_kernel: the row sums, accumulated chunk by chunk in the cache dtype as the
//      reference does, with the diagonal and the claimed entries taken out of their chunks.
// The softmax kernel then normalises the rows.

// One workgroup per valid page: 1 / norm of every key, claims reset to "none", and the sum of the
// normalised keys of every 16-key chunk of the page (fp32), which is all the row sums need:
//   sum_{j in chunk} e_i . e_j = e_i . (sum_{j in chunk} e_j).
// The reference walks the columns in chunks of 16 (BLOCK_N, raw_redudancy_score.py:176) and
// rounds after each chunk, so the chunk is the unit whose sum has to be exact.
template <typename T>
__global__ __launch_bounds__(kThreads) void raw_prep_kernel(GramArgs p) {
  static_assert(T::bytes == 2, "16-bit caches only");
  constexpr int PIECES = kDmax / 8, GROUPS = kThreads / PIECES;   // 16 groups of 16 lanes
  const int tid = threadIdx.x;
  const int piece = tid % PIECES, g = tid / PIECES;
  const int jp = blockIdx.x % p.NB;
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t obase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn + (int64_t)jp * p.BS;
  const float epsr = Elem<T>::rnd(p.eps);
  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) return;
  const bool pok = piece < p.D / 8;
  const int64_t k_row = (int64_t)p.Hkv * p.D * 2;
  const char* kbase = p.k + (l * p.k_sl + (int64_t)rpid * p.k_sp) * 2 + (int64_t)h * p.D * 2 +
                      (pok ? piece : 0) * 16;
  const int cpp = p.BS / kChunk;                       // chunks per page
  float* csum = p.ws_chunk + (obase / kChunk) * kDmax;  // [chunk][kDmax] of this page
  for (int c = g; c < cpp; c += GROUPS) {
    u32x4 raw[kChunk];
#pragma unroll
    for (int u = 0; u < kChunk; ++u)
      raw[u] = *(const u32x4*)(kbase + (int64_t)(c * kChunk + u) * k_row);
    float cs[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) cs[q] = 0.f;
#pragma unroll
    for (int u = 0; u < kChunk; ++u) {
      if (!pok) raw[u] = u32x4{0u, 0u, 0u, 0u};
      float e[8];
      Unpack<T>::run(vec16{raw[u].x, raw[u].y, raw[u].z, raw[u].w}, e);
      float ss = 0.f;
#pragma unroll
      for (int q = 0; q < 8; ++q) ss = fmaf(e[q], e[q], ss);
      ss = pieces_sum<PIECES>(ss);
      const float rn = __builtin_amdgcn_rcpf(fmaxf(Elem<T>::rnd(sqrtf(ss)), epsr));
#pragma unroll
      for (int q = 0; q < 8; ++q) cs[q] = fmaf(e[q], rn, cs[q]);
      if (piece == 0) {
        const int64_t oi = obase + c * kChunk + u;
        p.ws_sum[oi] = rn;      // kept for the row-sum kernel
        p.ws_val[oi] = rn;      // read by the Gram kernel, replaced by the claim values after it
        p.ws_col[oi] = -1;
      }
    }
    float* dst = csum + (int64_t)c * kDmax + piece * 8;
    *(float4*)dst = make_float4(cs[0], cs[1], cs[2], cs[3]);
    *(float4*)(dst + 4) = make_float4(cs[4], cs[5], cs[6], cs[7]);
  }
}

// Four waves per SIMD, i.e. two workgroups per compute unit (their LDS fits twice): one's barrier
// and LDS waits hide behind the other's tiles.  The register cap spills a few addresses outside
// the tile loop; measured 10-15 % faster than one workgroup per unit.
template <typename T, int TNc>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
void gram_raw_kernel(GramArgs p) {
  static_assert(T::bytes == 2, "16-bit caches only");
  typedef typename Mfma16<T>::V frag_t;
  constexpr int kThreads = 512, kWaves = 8;
  constexpr int PIECES = kDmax / 8;
  constexpr int ROWS_PER_IT = kThreads / PIECES;    // 32
  constexpr int STAGE_IT = TNc / ROWS_PER_IT;
  constexpr int NSUB = TNc / 32;
  constexpr int KSB = kDmax / 16;
  constexpr int PLANE = TNc * ROWH;

  extern __shared__ __align__(16) char smem[];
  char* buf0 = smem;                                // raw keys of a column tile
  char* buf1 = smem + PLANE;
  float* l_rn = (float*)(smem + 2 * PLANE);         // [2][TNc] 1 / norm of the tile's keys
  int* l_cside = (int*)(l_rn + 2 * TNc);            // [2][TNc] column-side claims of a tile
  float* l_rnrow = (float*)(l_cside + 2 * TNc);     // [BS] 1 / norm of the row page's keys
  int* vpage = (int*)(l_rnrow + p.BS);
  int* vidx = vpage + p.NB;
  __shared__ int nvalid_s, mine_s;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int jp = blockIdx.x % p.NB;
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t obase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn;

  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) return;
  list_valid_pages(p.table + (int64_t)b * p.NB, p.NB, p.num_pages, jp, vpage, vidx, nullptr, &nvalid_s, &mine_s);
  // head dims below 128 leave the upper pieces of every LDS row at zero
  for (int i = tid; i < 2 * PLANE / 4; i += kThreads) ((uint32_t*)smem)[i] = 0u;
  if (tid < 2 * TNc) l_cside[tid] = -1;
  for (int i = tid; i < p.BS; i += kThreads) l_rnrow[i] = p.ws_val[obase + (int64_t)jp * p.BS + i];
  __syncthreads();
  const int nv = nvalid_s, ia = mine_s;
  const int nd = nv / 2 + (((nv & 1) || ia < nv / 2) ? 1 : 0);   // page distances 0 .. nd-1
  const int tiles_per_page = p.BS / TNc;
  const int ntiles = nd * tiles_per_page;
  const int dpieces = p.D / 8;
  const int64_t k_row = (int64_t)p.Hkv * p.D * 2;
  const char* kbase = p.k + (l * p.k_sl) * 2 + (int64_t)h * p.D * 2;
  const float* rn_all = p.ws_val + obase;           // written by raw_prep_kernel

  const int st_piece = tid % PIECES, st_row0 = tid / PIECES;
  const bool st_ok = st_piece < dpieces;
  u32x4 pre[STAGE_IT];
  float pre_rn = 0.f;
  auto tile_page = [&](int tile, int& d, int& toff) {
    d = tile / tiles_per_page;
    toff = (tile - d * tiles_per_page) * TNc;
    const int ic = ia + d;
    return ic < nv ? ic : ic - nv;
  };
  auto issue_loads = [&](int tile) {
    int d, toff;
    const int ic = tile_page(tile, d, toff);
    const char* src = kbase + (int64_t)vpage[ic] * p.k_sp * 2 + (int64_t)toff * k_row +
                      (st_ok ? st_piece : 0) * 16;
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i)
      pre[i] = *(const u32x4*)(src + (int64_t)(st_row0 + i * ROWS_PER_IT) * k_row);
    if (tid < TNc) pre_rn = rn_all[vidx[ic] * p.BS + toff + tid];
  };
  auto commit_loads = [&](char* buf, int tile) {
    if (st_ok) {
#pragma unroll
      for (int i = 0; i < STAGE_IT; ++i)
        *(u32x4*)(buf + (st_row0 + i * ROWS_PER_IT) * ROWH + st_piece * 16) = pre[i];
    }
    if (tid < TNc) l_rn[(tile & 1) * TNc + tid] = pre_rn;
  };
  // Hands the column-side claims of a finished tile to the keys of its page and clears the slot.
  auto flush_cside = [&](int tile) {
    if (tid < TNc) {
      int d, toff;
      const int ic = tile_page(tile, d, toff);
      int* slot = l_cside + (tile & 1) * TNc + tid;
      const int v = *slot;
      if (v >= 0) {
        atomicMax(p.ws_col + obase + (int64_t)vidx[ic] * p.BS + toff + tid, v);
        *slot = -1;
      }
    }
  };
  const float thr_lo = p.threshold - fabsf(p.threshold) * 1e-5f - 1e-30f;

  const int row_blocks = p.BS / 32;
  const int NR = (row_blocks + kWaves - 1) / kWaves;
  for (int rr = 0; rr < NR; ++rr) {
    const int rb = rr * kWaves + wave;
    const bool active = rb < row_blocks;
    // ---- A fragments: this lane's key row as stored; lane (row, half) holds k = 16 s + 8 half + i
    frag_t ak[KSB];
    const float* rsrc = l_rnrow + (active ? rb : 0) * 32 + half * 4;   // this lane's 16 rows: 1 / norm
    {
      const int slot = (active ? rb : 0) * 32 + col;
      const char* src = kbase + (int64_t)rpid * p.k_sp * 2 + (int64_t)slot * k_row;
#pragma unroll
      for (int s = 0; s < KSB; ++s) {
        const int pc = 2 * s + half;
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (pc < dpieces) v = *(const u32x4*)(src + pc * 16);
        ak[s] = __builtin_bit_cast(frag_t, v);
      }
    }
    int dcol[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) dcol[r] = -1;

    if (ntiles > 0) { issue_loads(0); commit_loads(buf0, 0); }
    __syncthreads();
    for (int tile = 0; tile < ntiles; ++tile) {
      char* cur = (tile & 1) ? buf1 : buf0;
      char* nxt = (tile & 1) ? buf0 : buf1;
      if (tile + 1 < ntiles) issue_loads(tile + 1);
      if (tile > 0) flush_cside(tile - 1);   // its slot is next written two tiles from now
      int d, toff;
      const int ic = tile_page(tile, d, toff);
      const int jc = vidx[ic];
      if (active) {
#pragma unroll 1
        for (int st = 0; st < NSUB; ++st) {
          f32x16_t acc;
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = 0.f;
          const char* brow = cur + (st * 32 + col) * ROWH + half * 16;
          const float rn_col = l_rn[(tile & 1) * TNc + st * 32 + col];
#pragma unroll
          for (int s0 = 0; s0 < KSB; s0 += 4) {
            frag_t bk[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) bk[s] = *(const frag_t*)(brow + (s0 + s) * 32);
#pragma unroll
            for (int s = 0; s < 4; ++s) acc = Mfma16<T>::run(ak[s0 + s], bk[s], acc);
          }
          float rn_row[16];
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 v = *(const float4*)(rsrc + g * 8);
            rn_row[4 * g] = v.x; rn_row[4 * g + 1] = v.y; rn_row[4 * g + 2] = v.z; rn_row[4 * g + 3] = v.w;
          }
          const int cslot = toff + st * 32 + col;
          const int cidx = jc * p.BS + cslot;
          if (d == 0) {
            // the page against itself: a key against itself counts as 0
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3) == cslot) acc[r] = 0.f;
          }
          // most tiles hold no entry over the threshold: one maximum decides
          float big = -INFINITY;
#pragma unroll
          for (int r = 0; r < 16; ++r) big = fmaxf(big, acc[r] * rn_row[r]);
          if (!__any(big * rn_col > thr_lo)) continue;
          // row side: key (rb, r) sees column cidx; column side (other pages only: inside a
          // page both (i, j) and (j, i) are computed): key cidx sees the rows of this block,
          // whose index grows with r inside a lane
          int rlast = -1;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const bool over = acc[r] * (rn_row[r] * rn_col) > p.threshold;
            dcol[r] = max(dcol[r], over ? cidx : -1);
            rlast = over ? r : rlast;
          }
          if (d != 0 && __any(rlast >= 0)) {
            int ci = rlast < 0 ? -1
                               : jp * p.BS + rb * 32 + (rlast >> 2) * 8 + half * 4 + (rlast & 3);
            ci = max(ci, lane_xor32(ci));
            if (half == 0 && ci >= 0) atomicMax(&l_cside[(tile & 1) * TNc + st * 32 + col], ci);
          }
        }
      }
      if (tile + 1 < ntiles) commit_loads(nxt, tile + 1);
      __syncthreads();
    }
    if (ntiles > 0) flush_cside(ntiles - 1);
    bool any_mine = false;
#pragma unroll
    for (int r = 0; r < 16; ++r) any_mine |= dcol[r] >= 0;
    if (__any(any_mine)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = half_max_i(dcol[r]);
        if (active && col == 0 && c >= 0)
          atomicMax(p.ws_col + obase + (int64_t)jp * p.BS + rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3), c);
      }
    }
    __syncthreads();   // the claim slots are clear again before the next round writes them
  }
}

// The same for pages that are whole 128-key tiles, built like the page kernel of the lightning
// variant: four waves, each with TWO row blocks of the row page in registers (64 rows), so a B
// fragment read from LDS feeds two products; the column tiles go from global memory straight into
// LDS (wave w requests rows 32 w .. 32 w + 31 of a tile, the layout of `gram_page_kernel`), two
// buffers, one barrier per tile, the request for tile t + 1 under the products of tile t.  Two
// workgroups per compute unit (two waves per SIMD, 256 registers each).
constexpr int kRawTile = 128;
constexpr int kRawTileBytes = (kRawTile / 4) * kPgGrp;
template <typename T>
__global__ __launch_bounds__(256, 2) void gram_raw_wide_kernel(GramArgs p) {
  static_assert(T::bytes == 2, "16-bit caches only");
  typedef typename Mfma16<T>::V frag_t;
  constexpr int kThreads = 256, kWaves = 4, TNc = kRawTile;
  constexpr int PIECES = kDmax / 8;
  constexpr int NSUB = TNc / 32;
  constexpr int KSB = kDmax / 16;

  extern __shared__ __align__(16) char smem[];
  char* buf0 = smem;                                // raw keys of a column tile
  char* buf1 = smem + kRawTileBytes;
  float* l_rn = (float*)(smem + 2 * kRawTileBytes); // [2][TNc] 1 / norm of the tile's keys
  int* l_cside = (int*)(l_rn + 2 * TNc);            // [2][TNc] column-side claims of a tile
  float* l_rnrow = (float*)(l_cside + 2 * TNc);     // [BS] 1 / norm of the row page's keys
  int* vpage = (int*)(l_rnrow + p.BS);
  int* vidx = vpage + p.NB;
  __shared__ int nvalid_s, mine_s;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, col = lane & 31;
  const int jp = blockIdx.x % p.NB;
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t obase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn;

  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) return;
  list_valid_pages(p.table + (int64_t)b * p.NB, p.NB, p.num_pages, jp, vpage, vidx, nullptr, &nvalid_s, &mine_s);
  const int dpieces = p.D / 8;
  if (dpieces < PIECES) {   // head dims below 128 leave the upper pieces of every LDS row at zero
    for (int i = tid; i < 2 * kRawTileBytes / 4; i += kThreads) ((uint32_t*)smem)[i] = 0u;
  }
  if (tid < 2 * TNc) l_cside[tid] = -1;
  for (int i = tid; i < p.BS; i += kThreads) l_rnrow[i] = p.ws_val[obase + (int64_t)jp * p.BS + i];
  __syncthreads();
  const int nv = nvalid_s, ia = mine_s;
  const int nd = nv / 2 + (((nv & 1) || ia < nv / 2) ? 1 : 0);   // page distances 0 .. nd-1
  const int tiles_per_page = p.BS / TNc;
  const int ntiles = nd * tiles_per_page;
  const int k_row = p.Hkv * p.D * 2;
  const char* kbase = p.k + (l * p.k_sl) * 2 + (int64_t)h * p.D * 2;
  const float* rn_all = p.ws_val + obase;           // written by raw_prep_kernel

  auto tile_page = [&](int tile, int& d, int& toff) {
    d = tile / tiles_per_page;
    toff = (tile - d * tiles_per_page) * TNc;
    const int ic = ia + d;
    return ic < nv ? ic : ic - nv;
  };
  // tile -> LDS: eight instructions of four rows per wave; 1 / norm of the tile's keys to a register
  const int st_g = (lane >> 4) * 4 + (lane & 3), st_r = (lane >> 2) & 3;
  const int st_voff = st_r * k_row + st_g * 16;
  float pre_rn = 0.f;
  auto request = [&](int tile, char* buf) {
    int d, toff;
    const int ic = tile_page(tile, d, toff);
    const int pid = __builtin_amdgcn_readfirstlane(vpage[ic]);
    const char* src = kbase + (int64_t)pid * p.k_sp * 2 + (int64_t)(toff + wave * 32) * k_row;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, 32 * k_row, 0x00020000);
    if (st_g < dpieces) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)(buf + (wave * 8 + i) * kPgGrp), 16, st_voff,
                                                 i * 4 * k_row, 0, 0);
    }
    if (tid < TNc) pre_rn = rn_all[vidx[ic] * p.BS + toff + tid];
  };
  // Hands the column-side claims of a finished tile to the keys of its page and clears the slot.
  auto flush_cside = [&](int tile) {
    if (tid < TNc) {
      int d, toff;
      const int ic = tile_page(tile, d, toff);
      int* slot = l_cside + (tile & 1) * TNc + tid;
      const int v = *slot;
      if (v >= 0) {
        atomicMax(p.ws_col + obase + (int64_t)vidx[ic] * p.BS + toff + tid, v);
        *slot = -1;
      }
    }
  };
  const float thr_lo = p.threshold - fabsf(p.threshold) * 1e-5f - 1e-30f;
  // fragment of k-step s of this lane's row of a 32-row block: base + (s / 2) * 256 + (s % 2) * 32
  const int rd_off = (col >> 2) * kPgGrp + (col & 3) * 64 + half * 16;

  const int row_blocks = p.BS / 32;
  const int NR = (row_blocks + 2 * kWaves - 1) / (2 * kWaves);
  for (int rr = 0; rr < NR; ++rr) {
    const int rb0 = (rr * kWaves + wave) * 2;          // this wave's two row blocks: rb0, rb0 + 1
    const bool act0 = rb0 < row_blocks, act1 = rb0 + 1 < row_blocks;
    // ---- A fragments: this lane's two key rows as stored; lane (row, half) holds k = 16 s + 8 half + i
    frag_t ak0[KSB], ak1[KSB];
    {
      const char* src0 = kbase + (int64_t)rpid * p.k_sp * 2 + (int64_t)((act0 ? rb0 : 0) * 32 + col) * k_row;
      const char* src1 = kbase + (int64_t)rpid * p.k_sp * 2 + (int64_t)((act1 ? rb0 + 1 : 0) * 32 + col) * k_row;
#pragma unroll
      for (int s = 0; s < KSB; ++s) {
        const int pc = 2 * s + half;
        u32x4 v0 = u32x4{0u, 0u, 0u, 0u}, v1 = v0;
        if (pc < dpieces) {
          v0 = *(const u32x4*)(src0 + pc * 16);
          v1 = *(const u32x4*)(src1 + pc * 16);
        }
        ak0[s] = __builtin_bit_cast(frag_t, v0);
        ak1[s] = __builtin_bit_cast(frag_t, v1);
      }
    }
    float rn_row0[16], rn_row1[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 v0 = *(const float4*)(l_rnrow + (act0 ? rb0 : 0) * 32 + half * 4 + g * 8);
      const float4 v1 = *(const float4*)(l_rnrow + (act1 ? rb0 + 1 : 0) * 32 + half * 4 + g * 8);
      rn_row0[4 * g] = v0.x; rn_row0[4 * g + 1] = v0.y; rn_row0[4 * g + 2] = v0.z; rn_row0[4 * g + 3] = v0.w;
      rn_row1[4 * g] = v1.x; rn_row1[4 * g + 1] = v1.y; rn_row1[4 * g + 2] = v1.z; rn_row1[4 * g + 3] = v1.w;
    }
    int dcol0[16], dcol1[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { dcol0[r] = -1; dcol1[r] = -1; }

    if (ntiles > 0) request(0, buf0);
    for (int tile = 0; tile < ntiles; ++tile) {
      char* cur = (tile & 1) ? buf1 : buf0;
      char* nxt = (tile & 1) ? buf0 : buf1;
      // this wave's share of the tile (and its A fragments, the first time) has landed; after the
      // barrier so has everybody's, and everybody is done with the tile before
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (tid < TNc) l_rn[(tile & 1) * TNc + tid] = pre_rn;
      __syncthreads();
      if (tile + 1 < ntiles) request(tile + 1, nxt);
      if (tile > 0) flush_cside(tile - 1);   // its slot is next written two tiles from now
      int d, toff;
      const int ic = tile_page(tile, d, toff);
      const int jc = vidx[ic];
      // what a tile of 32 x 32 products feeds: the last column over the threshold of its rows and
      // (other pages only: inside a page both (i, j) and (j, i) are computed) the last row over
      // the threshold of its columns
      auto scan = [&](f32x16_t& acc, int rb, const float* rn_row, int* dcol, int st, float rn_col) {
        const int cslot = toff + st * 32 + col;
        const int cidx = jc * p.BS + cslot;
        if (d == 0) {
          // the page against itself: a key against itself counts as 0
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (rb * 32 + (r >> 2) * 8 + half * 4 + (r & 3) == cslot) acc[r] = 0.f;
        }
        // most tiles hold no entry over the threshold: one maximum decides
        float big = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) big = fmaxf(big, acc[r] * rn_row[r]);
        if (!__any(big * rn_col > thr_lo)) return;
        int rlast = -1;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const bool over = acc[r] * (rn_row[r] * rn_col) > p.threshold;
          dcol[r] = max(dcol[r], over ? cidx : -1);
          rlast = over ? r : rlast;
        }
        if (d != 0 && __any(rlast >= 0)) {
          int ci = rlast < 0 ? -1 : jp * p.BS + rb * 32 + (rlast >> 2) * 8 + half * 4 + (rlast & 3);
          ci = max(ci, lane_xor32(ci));
          if (half == 0 && ci >= 0) atomicMax(&l_cside[(tile & 1) * TNc + st * 32 + col], ci);
        }
      };
      if (act0) {
#pragma unroll 1
        for (int st = 0; st < NSUB; ++st) {
          f32x16_t acc0, acc1;
#pragma unroll
          for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
          const char* brow = cur + st * 8 * kPgGrp + rd_off;
          const float rn_col = l_rn[(tile & 1) * TNc + st * 32 + col];
#pragma unroll
          for (int s0 = 0; s0 < KSB; s0 += 4) {
            frag_t bk[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) bk[s] = *(const frag_t*)(brow + ((s0 + s) >> 1) * 256 + ((s0 + s) & 1) * 32);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              acc0 = Mfma16<T>::run(ak0[s0 + s], bk[s], acc0);
              acc1 = Mfma16<T>::run(ak1[s0 + s], bk[s], acc1);
            }
          }
          scan(acc0, rb0, rn_row0, dcol0, st, rn_col);
          if (act1) scan(acc1, rb0 + 1, rn_row1, dcol1, st, rn_col);
        }
      }
    }
    __syncthreads();   // everybody is done with the last tile
    if (ntiles > 0) flush_cside(ntiles - 1);
    bool any_mine = false;
#pragma unroll
    for (int r = 0; r < 16; ++r) any_mine |= dcol0[r] >= 0 || dcol1[r] >= 0;
    if (__any(any_mine)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c0 = half_max_i(dcol0[r]), c1 = half_max_i(dcol1[r]);
        const int64_t row = obase + (int64_t)jp * p.BS + rb0 * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
        if (act0 && col == 0 && c0 >= 0) atomicMax(p.ws_col + row, c0);
        if (act1 && col == 0 && c1 >= 0) atomicMax(p.ws_col + row + 32, c1);
      }
    }
    __syncthreads();   // the claim slots are clear again before the next round writes them
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void raw_claim_value_kernel(GramArgs p) {
  static_assert(T::bytes == 2, "16-bit caches only");
  constexpr int PIECES = kDmax / 8, GROUPS = kThreads / PIECES;
  const int tid = threadIdx.x;
  const int piece = tid % PIECES, g = tid / PIECES;
  const int jp = blockIdx.x % p.NB;
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t obase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn;
  const float epsr = Elem<T>::rnd(p.eps);
  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) return;
  const bool pok = piece < p.D / 8;
  const int64_t k_row = (int64_t)p.Hkv * p.D * 2;
  const char* kbase = p.k + (l * p.k_sl) * 2 + (int64_t)h * p.D * 2 + (pok ? piece : 0) * 16;
  for (int slot = g; slot < p.BS; slot += GROUPS) {
    const int64_t oi = obase + (int64_t)jp * p.BS + slot;
    const int c = p.ws_col[oi];
    if (c < 0 || c >= Tn) continue;     // uniform over the 16 lanes of a key
    if (c == jp * p.BS + slot) {        // negative threshold: the zeroed diagonal entry was claimed
      if (piece == 0) p.ws_val[oi] = 0.f;
      continue;
    }
    const int cp = c / p.BS, cs = c - cp * p.BS;
    const int ccode = p.table[(int64_t)b * p.NB + cp];
    const int cpid = page_is_pad(ccode) ? -1 : page_id(ccode);
    if (cpid < 0 || cpid >= p.num_pages) continue;
    u32x4 ra = *(const u32x4*)(kbase + (int64_t)rpid * p.k_sp * 2 + (int64_t)slot * k_row);
    u32x4 rc = *(const u32x4*)(kbase + (int64_t)cpid * p.k_sp * 2 + (int64_t)cs * k_row);
    if (!pok) { ra = u32x4{0u, 0u, 0u, 0u}; rc = ra; }
    float ea[8], ec[8];
    Unpack<T>::run(vec16{ra.x, ra.y, ra.z, ra.w}, ea);
    Unpack<T>::run(vec16{rc.x, rc.y, rc.z, rc.w}, ec);
    float sa = 0.f, sc = 0.f, t = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      sa = fmaf(ea[q], ea[q], sa);
      sc = fmaf(ec[q], ec[q], sc);
      t = fmaf(ea[q], ec[q], t);
    }
    sa = pieces_sum<PIECES>(sa);
    sc = pieces_sum<PIECES>(sc);
    t = pieces_sum<PIECES>(t);
    const float rna = __builtin_amdgcn_rcpf(fmaxf(Elem<T>::rnd(sqrtf(sa)), epsr));
    const float rnc = __builtin_amdgcn_rcpf(fmaxf(Elem<T>::rnd(sqrtf(sc)), epsr));
    if (piece == 0) p.ws_val[oi] = t * rna * rnc;
  }
}

// ------------------------------------------------------------------ raw, 16-bit: row sums
// The reference accumulates a key's row sum in the CACHE dtype: per column page one partial sum,
// rounded after each 16-column chunk (raw_redudancy_score.py:146-155: load, add the chunk's fp32
// sum, store in the cache dtype), then the partial sums of the pages are added in fp32 and rounded
// once (:218, torch.sum).  This kernel restates that chain exactly.
//   chunk sum   c(i, chunk) = rn_i (k_i . s_chunk) - [i in chunk] S_ii - sum_{j in chunk, claimed by i} S_ij
// with s_chunk the sum of the chunk's normalised keys from raw_prep_kernel.  The dot products of
// a page's 256 keys with 32 chunks at a time run on the matrix cores: the keys as stored (exact
// 16-bit products), s_chunk split into three 16-bit planes (together its full fp32 mantissa).
// One workgroup per valid page; wave w owns keys 32 w .. 32 w + 31.
// chunk sums are below 16 + 1 in magnitude: 2^-26 fixed point fits 32 bits, and integer atomics
// make the sum of several claims independent of their order
__device__ __forceinline__ int to_fixed26(float v) { return (int)(v * 67108864.f); }
__device__ __forceinline__ float from_fixed26(int w) { return (float)w * (1.f / 67108864.f); }

#ifdef ZP_PAGE_STAMP
__device__ long long zp_chain_stamp_buf[(1 << 16) * 12];
extern "C" int zp_debug_chain_stamps(long long* dst, int n_groups) {
  return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(zp_chain_stamp_buf), (size_t)n_groups * 12 * 8);
}
#define ZP_CSTAMP(i) do { if (tid == 0) { const long long c_ = clock64(); acc_[i] += c_ - last_; last_ = c_; } } while (0)
#else
#define ZP_CSTAMP(i) do { } while (0)
#endif

template <typename T>
__global__ __launch_bounds__(512, 4) void raw_chain_kernel(GramArgs p) {
  static_assert(T::bytes == 2, "16-bit caches only");
  typedef typename Mfma16<T>::V frag_t;
  constexpr int kT = 512, kW = 8, KSB = kDmax / 16, CT = 32;     // CT chunks per tile
  constexpr int KEYS = kW * 32;                                     // keys per round
  extern __shared__ __align__(16) char smem[];
  char* planes = smem;                                   // [3][CT] rows of ROWH bytes
  int* cl = (int*)(smem + 3 * CT * ROWH);                // [CT][KEYS] corrections, then chunk sums
  int* vidx = cl + CT * KEYS;                            // [NB] logical page of the n-th valid page
  int* vord = vidx + p.NB;                               // [NB] inverse (-1: pad)
  // the claims taken from this round's keys, gathered once per round: (chunk << 16 | key) and value
  uint32_t* lst_key = (uint32_t*)(vord + p.NB);          // [NB * BS]
  float* lst_val = (float*)(lst_key + (size_t)p.NB * p.BS);
  __shared__ int nvalid_s, nlist_s;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
#ifdef ZP_PAGE_STAMP
  long long acc_[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  long long last_ = clock64();
  const long long wall0 = wall_clock64();
#endif
  const int jp = blockIdx.x % p.NB;
  const int h = (blockIdx.x / p.NB) % p.Hkv;
  const int b = (blockIdx.x / (p.NB * p.Hkv)) % p.B;
  const int l = blockIdx.x / (p.NB * p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t obase = (((int64_t)l * p.B + b) * p.Hkv + h) * Tn;

  const int code = p.table[(int64_t)b * p.NB + jp];
  int rpid = page_is_pad(code) ? -1 : page_id(code);
  if (rpid >= p.num_pages) rpid = -1;
  if (rpid < 0) {
    for (int s = tid; s < p.BS; s += kT) Elem<T>::st(p.r_out, obase + (int64_t)jp * p.BS + s, -INFINITY);
    return;
  }
  list_valid_pages(p.table + (int64_t)b * p.NB, p.NB, p.num_pages, jp, nullptr, vidx, vord, &nvalid_s, nullptr);
  __syncthreads();
  const int cpp = p.BS / kChunk;
  const int nchunks = nvalid_s * cpp;
  const int ntiles = (nchunks + CT - 1) / CT;
  const int my_ord = vord[jp];
  const int dpieces = p.D / 8;
  const int64_t k_row = (int64_t)p.Hkv * p.D * 2;
  const char* kpage = p.k + (l * p.k_sl + (int64_t)rpid * p.k_sp) * 2 + (int64_t)h * p.D * 2;
  const float* chunk_all = p.ws_chunk + (obase / kChunk) * kDmax;

  const int rounds = (p.BS + KEYS - 1) / KEYS;
  for (int rr = 0; rr < rounds; ++rr) {
    const int key0 = rr * KEYS;                       // first slot of this round
    const int slot = key0 + wave * 32 + col;          // this lane's key (both halves of the wave)
    const bool live = slot < p.BS;
    // ---- B fragments: the key as stored; lane (key, half) holds k = 16 s + 8 half + i
    frag_t bk[KSB];
    float ssq = 0.f;
    {
      const char* src = kpage + (int64_t)(live ? slot : 0) * k_row;
#pragma unroll
      for (int s = 0; s < KSB; ++s) {
        const int pc = 2 * s + half;
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (live && pc < dpieces) v = *(const u32x4*)(src + pc * 16);
        bk[s] = __builtin_bit_cast(frag_t, v);
        float e[8];
        Unpack<T>::run(vec16{v.x, v.y, v.z, v.w}, e);
#pragma unroll
        for (int q = 0; q < 8; ++q) ssq = fmaf(e[q], e[q], ssq);
      }
      ssq += lane_xor32(ssq);
    }
    ZP_CSTAMP(0);   // set-up, key loads issued
    const float rn = live ? p.ws_sum[obase + (int64_t)jp * p.BS + slot] : 0.f;
    const float diag = ssq * rn * rn;                 // S_ii, the entry the reference zeroes
    const int own_chunk = my_ord * cpp + slot / kChunk;
    float part = 0.f, total = 0.f;                    // chain state of key `tid` (tid < KEYS)
    // every key of the sequence claims at most one entry: one pass over the claims keeps those
    // taken from this round's keys, with the chunk of the claiming key (the order of the list does
    // not matter, the values are added as fixed point)
    __syncthreads();
    if (tid == 0) nlist_s = 0;
    __syncthreads();
    for (int t0 = tid; t0 < Tn; t0 += 4 * kT) {      // four independent loads in flight per thread
      int cw[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * kT;
        cw[u] = t < Tn ? p.ws_col[obase + t] : -1;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * kT;
        if (t >= Tn) continue;
        const int jt = t / p.BS;
        const int ord = vord[jt];
        if (ord < 0) continue;
        const int cc = cw[u] - (jp * p.BS + key0);   // the row key t claimed from
        if (cc >= 0 && cc < KEYS && key0 + cc < p.BS) {
          const int i = atomicAdd(&nlist_s, 1);
          lst_key[i] = (uint32_t)(ord * cpp + (t - jt * p.BS) / kChunk) << 16 | (uint32_t)cc;
          lst_val[i] = p.ws_val[obase + t];
        }
      }
    }
    __syncthreads();
    const int nlist = nlist_s;
    ZP_CSTAMP(1);   // claims gathered

    // the chunk sums of a tile (CT chunks x kDmax floats, two float4 per thread) are requested one
    // tile ahead and split into the three planes once the tile before is done with them
    static_assert(CT * (kDmax / 4) == 2 * kT, "two float4 of a tile's chunk sums per thread");
    float4 pv[2];
    auto request_planes = [&](int tile) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int i = tid + u * kT;
        const int m = i / (kDmax / 4), q4 = i - m * (kDmax / 4);
        const int vc = tile * CT + m;
        pv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (vc < nchunks) {
          const int vp = vc / cpp, c = vc - vp * cpp;
          pv[u] = *(const float4*)(chunk_all + ((int64_t)vidx[vp] * cpp + c) * kDmax + q4 * 4);
        }
      }
    };
    auto store_planes = [&]() {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int i = tid + u * kT;
        const int m = i / (kDmax / 4), q4 = i - m * (kDmax / 4);
        const float f[4] = {pv[u].x, pv[u].y, pv[u].z, pv[u].w};
        uint16_t o[4][3];
#pragma unroll
        for (int q = 0; q < 4; ++q) Split3<T>::run(f[q], o[q]);
#pragma unroll
        for (int pl = 0; pl < 3; ++pl) {
          uint2 w;
          w.x = (uint32_t)o[0][pl] | ((uint32_t)o[1][pl] << 16);
          w.y = (uint32_t)o[2][pl] | ((uint32_t)o[3][pl] << 16);
          *(uint2*)(planes + (pl * CT + m) * ROWH + q4 * 8) = w;
        }
      }
    };
    if (ntiles > 0) { request_planes(0); store_planes(); }
    if (ntiles > 1) request_planes(1);
    ZP_CSTAMP(2);   // first planes
    for (int tile = 0; tile < ntiles; ++tile) {
      const int c0 = tile * CT;
      // ---- corrections of this tile (its three planes are in LDS)
      for (int i = tid; i < CT * KEYS / 4; i += kT) ((int4*)cl)[i] = make_int4(0, 0, 0, 0);
      __syncthreads();
      ZP_CSTAMP(3);   // corrections cleared
      if (half == 0 && live && own_chunk >= c0 && own_chunk < c0 + CT)
        atomicAdd(&cl[(own_chunk - c0) * KEYS + wave * 32 + col], to_fixed26(diag));
      for (int i = tid; i < nlist; i += kT) {
        const uint32_t w = lst_key[i];
        const int vc = (int)(w >> 16);
        if (vc >= c0 && vc < c0 + CT)
          atomicAdd(&cl[(vc - c0) * KEYS + (int)(w & 0xffffu)], to_fixed26(lst_val[i]));
      }
      __syncthreads();
      ZP_CSTAMP(4);   // corrections added
      // ---- chunk sums of the tile: A = planes (rows = chunks), B = keys
      {
        f32x16_t acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int pl = 2; pl >= 0; --pl) {
          const char* arow = planes + (pl * CT + col) * ROWH + half * 16;
#pragma unroll
          for (int s = 0; s < KSB; ++s) acc = Mfma16<T>::run(*(const frag_t*)(arow + s * 32), bk[s], acc);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = (r >> 2) * 8 + half * 4 + (r & 3);
          int* slot_p = &cl[m * KEYS + wave * 32 + col];
          *slot_p = __float_as_int(acc[r] * rn - from_fixed26(*slot_p));
        }
      }
      __syncthreads();
      ZP_CSTAMP(5);   // products
      // the products are done with this tile's planes: the next tile's go in, the one after is requested
      if (tile + 1 < ntiles) {
        store_planes();
        if (tile + 2 < ntiles) request_planes(tile + 2);
      }
      // ---- the reference's chain: one cache-dtype partial sum per column page
      if (tid < KEYS) {
        int cm = c0 % cpp;                     // where the tile's first chunk lies inside its page
        const int mend = min(CT, nchunks - c0);
        for (int m0 = 0; m0 < mend; m0 += 8) {   // eight chunk sums read ahead of the serial chain
          float v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) v[u] = m0 + u < mend ? __int_as_float(cl[(m0 + u) * KEYS + tid]) : 0.f;
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            if (m0 + u < mend) {
              if (cm == 0) { total += part; part = 0.f; }
              part = Elem<T>::rnd(part + v[u]);
              cm = cm + 1 == cpp ? 0 : cm + 1;
            }
          }
        }
      }
      ZP_CSTAMP(6);   // next planes stored, chain of thread 0
      __syncthreads();
      ZP_CSTAMP(7);   // barrier behind the chain
    }
    if (tid < KEYS && key0 + tid < p.BS)
      Elem<T>::st(p.r_out, obase + (int64_t)jp * p.BS + key0 + tid, total + part);
  }
#ifdef ZP_PAGE_STAMP
  if (tid == 0 && blockIdx.x < (1 << 16)) {
    long long* dst = zp_chain_stamp_buf + (int64_t)blockIdx.x * 12;
    for (int i = 0; i < 8; ++i) dst[i] = acc_[i];
    dst[10] = wall0;
    dst[11] = wall_clock64() - wall0;
  }
#endif
}
#undef ZP_CSTAMP

// ------------------------------------------------------------------ softmax epilogue
// One workgroup per (layer, sequence, head) row of T logits:
//   raw only: r_i = rowsum_i - sum_{j: c*(j)=i} v_j, pad pages -inf
//   x = rnd(r / divisor); x = rnd(x - max); out = rnd(exp(x) / sum)
__device__ __forceinline__ float block_reduce(float v, float* lds, bool is_max) {
  if (is_max) v = wave_max(v); else v = wave_sum(v);
  __syncthreads();
  if (lane_id() == 0) lds[wave_id()] = v;
  __syncthreads();
  float m = lds[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) m = is_max ? fmaxf(m, lds[i]) : m + lds[i];
  return m;
}

template <typename T, bool RAW>
__global__ __launch_bounds__(kThreads) void red_softmax_kernel(
    void* __restrict__ red, void* __restrict__ logits, const int32_t* __restrict__ table,
    const float* __restrict__ ws_sum, const int32_t* __restrict__ ws_col,
    const float* __restrict__ ws_val, int B, int NB, int BS, int Hkv, int num_pages,
    float tscale /* raw: temperature; lightning: temperature*BS */,
    int rows_ready /* raw: the row sums are already in `red` (16-bit caches) */,
    const float* __restrict__ ws_csum = nullptr /* raw, fp32, every pair of pages once: column-side
        sums [distance - 1][row][Tn]; ws_col then holds 64-bit (index + 1, value) claims */,
    int64_t n_keys = 0) {
  extern __shared__ __align__(16) char smem[];
  __shared__ float red_lds[kWaves];
  const int Tn = NB * BS;
  // raw: [Tn] 64-bit sums of the values claimed from each row, then the [Tn] floats of the row
  unsigned long long* corr = (unsigned long long*)smem;
  const bool from_ws = RAW && !rows_ready;
  float* x = (float*)(smem + (from_ws ? (size_t)Tn * 8 : 0));
  const int64_t row = blockIdx.x;
  const int b = (int)((row / Hkv) % B);
  const int64_t base = row * Tn;
  const int32_t* trow = table + (int64_t)b * NB;
  int nvalid = 0;
  for (int j = 0; j < NB; ++j) {
    const int c = trow[j];
    const int pid = page_is_pad(c) ? -1 : page_id(c);
    nvalid += (pid >= 0 && pid < num_pages) ? 1 : 0;
  }
  const float divisor = RAW ? tscale * (float)(nvalid * BS) : tscale;
  const unsigned long long* claims = (const unsigned long long*)ws_col;
  if (from_ws) {
    // every key hands the value of its claimed entry to the row it was taken from: 2^-32 fixed
    // point with integer atomics, exact and independent of the order
    for (int t = threadIdx.x; t < Tn; t += kThreads) corr[t] = 0ull;
    __syncthreads();
    for (int t = threadIdx.x; t < Tn; t += kThreads) {
      const int c = trow[t / BS];
      const int pid = page_is_pad(c) ? -1 : page_id(c);
      if (pid < 0 || pid >= num_pages) continue;
      if (ws_csum) {
        const unsigned long long cl = claims[base + t];
        const int cc = (int)(cl >> 32) - 1;
        if (cc >= 0 && cc < Tn) atomicAdd(&corr[cc], to_fixed32(__uint_as_float((unsigned)cl)));
      } else {
        const int cc = ws_col[base + t];
        if (cc >= 0 && cc < Tn) atomicAdd(&corr[cc], to_fixed32(ws_val[base + t]));
      }
    }
    __syncthreads();
  }
  float mloc = -INFINITY;
  for (int t = threadIdx.x; t < Tn; t += kThreads) {
    float r;
    if (from_ws) {
      const int c = trow[t / BS];
      const int pid = page_is_pad(c) ? -1 : page_id(c);
      if (pid >= 0 && pid < num_pages) {
        float sv = ws_sum[base + t];
        if (ws_csum) {
          // the column-side sums of this key's page: distance d was written by the valid page
          // d places before it (cyclically), if that page ran the distance
          int ci = 0;
          for (int j = 0; j < t / BS; ++j) {
            const int c2 = trow[j];
            const int p2 = page_is_pad(c2) ? -1 : page_id(c2);
            ci += (p2 >= 0 && p2 < num_pages) ? 1 : 0;
          }
          for (int d = 1; d <= nvalid / 2; ++d) {
            const int a = ci - d >= 0 ? ci - d : ci - d + nvalid;
            const bool ran = d < nvalid / 2 + (((nvalid & 1) || a < nvalid / 2) ? 1 : 0);
            if (ran) sv += ws_csum[(int64_t)(d - 1) * n_keys + base + t];
          }
        }
        r = Elem<T>::rnd(sv - from_fixed32(corr[t]));
      } else {
        r = -INFINITY;
      }
    } else {
      r = Elem<T>::ld(red, base + t);
    }
    if (logits) Elem<T>::st(logits, base + t, r);
    const float xv = Elem<T>::rnd(r / divisor);
    x[t] = xv;
    mloc = fmaxf(mloc, xv);
  }
  const float m = block_reduce(mloc, red_lds, true);
  float sloc = 0.f;
  for (int t = threadIdx.x; t < Tn; t += kThreads) {
    const float e = expf(Elem<T>::rnd(x[t] - m));
    x[t] = e;
    sloc += e;
  }
  const float ssum = block_reduce(sloc, red_lds, false);
  for (int t = threadIdx.x; t < Tn; t += kThreads) Elem<T>::st(red, base + t, x[t] / ssum);
}

int check_common(const char* name, const void* k_cache, const int32_t* table, void* red_out,
                 int L, int B, int NB, int BS, int Hkv, int D, int dtype, int64_t k_sl,
                 int64_t k_sp) {
  ZP_REQUIRE(k_cache && table && red_out, "%s: null pointer", name);
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0 && D > 0, "%s: bad dims", name);
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "%s: unknown dtype tag %d", name, dtype);
  const int es = zp_dtype_bytes(dtype);
  if (!(D <= kDmax && (D * es) % 16 == 0)) {
    zp_set_error("%s: head_dim %d unsupported (need <= %d and a multiple of %d)", name, D, kDmax,
                 16 / es);
    return ZP_EUNSUPPORTED;
  }
  if (BS % TN != 0) {
    zp_set_error("%s: page size %d is not a multiple of %d", name, BS, TN);
    return ZP_EUNSUPPORTED;
  }
  ZP_REQUIRE(((uintptr_t)k_cache % 16) == 0 && (k_sl * es) % 16 == 0 && (k_sp * es) % 16 == 0,
             "%s: key cache must be 16-byte aligned", name);
  return ZP_OK;
}

// fp32 all-pairs: can every unordered pair of pages be multiplied once (pages of at most 256
// keys in whole 64-key tiles, column-sum slots for every distance in the workspace)?
inline bool raw_f32_symmetric(int NB, int BS) {
  return BS <= 256 && BS % TN == 0 && NB / 2 <= kSymMaxDist;
}

template <typename T, bool RAW>
int launch_gram(const GramArgs& a, int L, hipStream_t st) {
  dim3 grid((unsigned)((int64_t)L * a.B * a.Hkv * a.NB));
  const size_t tail = (RAW ? 0 : (size_t)a.BS * 20) + sizeof(int) * 2 * a.NB;
  if constexpr (T::bytes == 2 && !RAW) {
    // one workgroup per (layer, sequence, kv head) row; the block table row sits in LDS
    const size_t smem = (size_t)kPgBytes + 4 * kDmax * 2 + 4 * kPageRows * 2 +
                        (size_t)kPageRows * (2 * 8 + 2 * 4 + 4 + 4) + sizeof(int) * (kPageWaves + a.NB);
    if (a.BS <= kPageRows && a.BS % 32 == 0 && smem <= 80 * 1024) {
      grid = dim3((unsigned)((int64_t)L * a.B * a.Hkv));
      if (hipFuncSetAttribute((const void*)gram_page_kernel<T>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
        zp_set_error("redundancy: cannot reserve %zu bytes of LDS", smem);
        return ZP_EHIP;
      }
      hipLaunchKernelGGL((gram_page_kernel<T>), grid, dim3(kPageThreads), smem, st, a);
      ZP_LAUNCH_CHECK();
      return ZP_OK;
    }
  }
  if constexpr (T::bytes == 4 && !RAW) {
    if (a.BS <= kPage32Rows && a.BS % 32 == 0 && a.NB <= 1024) {
      // one workgroup per (layer, sequence, kv head) row
      grid = dim3((unsigned)((int64_t)L * a.B * a.Hkv));
      const size_t smem = (size_t)kPage32Rows * ROWF * 4 + (size_t)kPage32Rows * (8 + 8 + 4 + 4 * 4) +
                          sizeof(int) * a.NB;
      if (hipFuncSetAttribute((const void*)gram_page_f32_kernel,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
        zp_set_error("redundancy: cannot reserve %zu bytes of LDS", smem);
        return ZP_EHIP;
      }
      hipLaunchKernelGGL(gram_page_f32_kernel, grid, dim3(kPage32Threads), smem, st, a);
      ZP_LAUNCH_CHECK();
      return ZP_OK;
    }
  }
  if constexpr (T::bytes == 4 && RAW) {
    if (raw_f32_symmetric(a.NB, a.BS)) {
      const int64_t n = (int64_t)L * a.B * a.Hkv * a.NB * a.BS;
      const size_t smem = sizeof(float) * (2 * TN * ROWF + 2 * kSymWaves * TN) + sizeof(int) * 2 * a.NB;
      if (hipFuncSetAttribute((const void*)gram_raw_sym_f32_kernel,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
        zp_set_error("redundancy: cannot reserve %zu bytes of LDS", smem);
        return ZP_EHIP;
      }
      hipLaunchKernelGGL(fill_u64_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                         (unsigned long long*)a.ws_col, n, 0ull);
      hipLaunchKernelGGL(gram_raw_sym_f32_kernel, grid, dim3(kSymWaves * 64), smem, st, a);
      ZP_LAUNCH_CHECK();
      return ZP_OK;
    }
  }
  if constexpr (T::bytes == 2 && RAW) {
    // column tiles of 128 keys when the page size allows: half as many workgroup barriers
    const int tn = a.BS % 128 == 0 ? 128 : TN;
    const size_t smem1 = 2 * (size_t)tn * ROWH + sizeof(int) * 4 * tn + sizeof(float) * a.BS +
                         sizeof(int) * 2 * a.NB;
    const void* fn = tn == 128 ? (const void*)gram_raw_kernel<T, 128> : (const void*)gram_raw_kernel<T, TN>;
    // whole 128-key tiles: the four-wave kernel with two row blocks per wave
    const size_t smemw = 2 * (size_t)kRawTileBytes + sizeof(int) * 4 * kRawTile + sizeof(float) * a.BS +
                         sizeof(int) * 2 * a.NB;
    const bool wide = tn == 128 && smemw <= 80 * 1024;
    const size_t smem2 = 3 * 32 * (size_t)ROWH + sizeof(int) * 32 * 256 + sizeof(int) * 2 * a.NB +
                         (size_t)a.NB * a.BS * 8;   // + the round's claim list
    if (smem2 > 160 * 1024) {
      zp_set_error("redundancy: a row of %d tokens exceeds LDS", a.NB * a.BS);
      return ZP_EUNSUPPORTED;
    }
    if (hipFuncSetAttribute(wide ? (const void*)gram_raw_wide_kernel<T> : fn,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)(wide ? smemw : smem1)) != hipSuccess ||
        hipFuncSetAttribute((const void*)raw_chain_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem2) != hipSuccess) {
      zp_set_error("redundancy: cannot reserve %zu / %zu bytes of LDS", smem1, smem2);
      return ZP_EHIP;
    }
    hipLaunchKernelGGL((raw_prep_kernel<T>), grid, dim3(kThreads), 0, st, a);
    if (wide) hipLaunchKernelGGL((gram_raw_wide_kernel<T>), grid, dim3(256), smemw, st, a);
    else if (tn == 128) hipLaunchKernelGGL((gram_raw_kernel<T, 128>), grid, dim3(512), smem1, st, a);
    else hipLaunchKernelGGL((gram_raw_kernel<T, TN>), grid, dim3(512), smem1, st, a);
    hipLaunchKernelGGL((raw_claim_value_kernel<T>), grid, dim3(kThreads), 0, st, a);
    hipLaunchKernelGGL((raw_chain_kernel<T>), grid, dim3(512), smem2, st, a);
    ZP_LAUNCH_CHECK();
    return ZP_OK;
  }
  if constexpr (T::bytes == 2 && !RAW) {
    const size_t smem = 4 * (size_t)TN * ROWH + tail;
    const bool wide = a.BS / 32 > kWaves;   // more row blocks than 4 waves: use 8 and halve the passes
    const void* fn = wide ? (const void*)gram_split_kernel<T, RAW, 8> : (const void*)gram_split_kernel<T, RAW, 4>;
    if (smem > 64 * 1024 &&
        hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      zp_set_error("redundancy: cannot reserve %zu bytes of LDS", smem);
      return ZP_EHIP;
    }
    if (wide) hipLaunchKernelGGL((gram_split_kernel<T, RAW, 8>), grid, dim3(512), smem, st, a);
    else hipLaunchKernelGGL((gram_split_kernel<T, RAW, 4>), grid, dim3(kThreads), smem, st, a);
  } else {
    const size_t smem = sizeof(float) * 2 * TN * ROWF + tail;
    // more row blocks than 4 waves: 8 waves take the page's rows in one pass, so every column
    // tile is staged (and normalised) once instead of twice
    const bool wide = a.BS / 32 > kWaves;
    const void* fn = wide ? (const void*)gram_kernel<T, RAW, 8> : (const void*)gram_kernel<T, RAW, 4>;
    if (smem > 64 * 1024 &&
        hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      zp_set_error("redundancy: cannot reserve %zu bytes of LDS", smem);
      return ZP_EHIP;
    }
    if (wide) hipLaunchKernelGGL((gram_kernel<T, RAW, 8>), grid, dim3(512), smem, st, a);
    else hipLaunchKernelGGL((gram_kernel<T, RAW, 4>), grid, dim3(kThreads), smem, st, a);
  }
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

template <typename T, bool RAW>
int launch_softmax(void* red, void* logits, const int32_t* table, const float* ws_sum,
                   const int32_t* ws_col, const float* ws_val, int L, int B, int NB, int BS,
                   int Hkv, int num_pages, double temperature, hipStream_t st, int rows_ready = 0,
                   const float* ws_csum = nullptr) {
  const size_t smem = (size_t)NB * BS * ((RAW && !rows_ready) ? 12 : 4);
  if (smem > 150 * 1024) {
    zp_set_error("redundancy: a row of %d tokens exceeds LDS", NB * BS);
    return ZP_EUNSUPPORTED;
  }
  if (smem > 64 * 1024 &&
      hipFuncSetAttribute((const void*)red_softmax_kernel<T, RAW>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    zp_set_error("redundancy: cannot reserve %zu bytes of LDS", smem);
    return ZP_EHIP;
  }
  dim3 grid((unsigned)((int64_t)L * B * Hkv));
  hipLaunchKernelGGL((red_softmax_kernel<T, RAW>), grid, dim3(kThreads), smem, st, red, logits,
                     table, ws_sum, ws_col, ws_val, B, NB, BS, Hkv, num_pages,
                     RAW ? (float)temperature : (float)(temperature * (double)BS), rows_ready,
                     ws_csum, (int64_t)L * B * Hkv * NB * BS);
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

}  // namespace

extern "C" int zp_redundancy_lightning(const void* k_cache, const int32_t* block_table,
                                       void* red_out, void* logits_out, int32_t L, int32_t B,
                                       int32_t NB, int32_t BS, int32_t Hkv, int32_t D,
                                       int32_t num_pages, int64_t k_sl, int64_t k_sp,
                                       float threshold, double temperature, int32_t dtype,
                                       void* stream) {
  int rc = check_common("redundancy_lightning", k_cache, block_table, red_out, L, B, NB, BS, Hkv,
                        D, dtype, k_sl, k_sp);
  if (rc != ZP_OK) return rc;
  if (L == 0 || B == 0) return ZP_OK;
  GramArgs a;
  a.k = (const char*)k_cache; a.table = block_table; a.r_out = red_out;
  a.ws_sum = nullptr; a.ws_col = nullptr; a.ws_val = nullptr; a.ws_chunk = nullptr;
  a.B = B; a.NB = NB; a.BS = BS; a.Hkv = Hkv; a.D = D; a.num_pages = num_pages;
  a.k_sl = k_sl; a.k_sp = k_sp; a.threshold = threshold; a.eps = 1e-6f;
  hipStream_t st = (hipStream_t)stream;
  ZP_DISPATCH_DTYPE(dtype, {
    rc = launch_gram<T, false>(a, L, st);
    if (rc != ZP_OK) return rc;
    rc = launch_softmax<T, false>(red_out, logits_out, block_table, nullptr, nullptr, nullptr, L,
                                  B, NB, BS, Hkv, num_pages, temperature, st);
  });
  return rc;
}

extern "C" int64_t zp_redundancy_raw_workspace(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                               int32_t Hkv) {
  // three fp32 / int32 words per key, and for 16-bit caches kDmax floats per chunk of 16 keys
  return (int64_t)L * B * Hkv * NB * BS * (12 + 4 * kDmax / kChunk);
}

extern "C" int zp_redundancy_raw(const void* k_cache, const int32_t* block_table, void* red_out,
                                 void* logits_out, int32_t L, int32_t B, int32_t NB, int32_t BS,
                                 int32_t Hkv, int32_t D, int32_t num_pages, int64_t k_sl,
                                 int64_t k_sp, float threshold, double temperature, int32_t dtype,
                                 void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = check_common("redundancy_raw", k_cache, block_table, red_out, L, B, NB, BS, Hkv, D,
                        dtype, k_sl, k_sp);
  if (rc != ZP_OK) return rc;
  if (L == 0 || B == 0) return ZP_OK;
  const int64_t n = (int64_t)L * B * Hkv * NB * BS;
  const int64_t need = zp_redundancy_raw_workspace(L, B, NB, BS, Hkv);
  ZP_REQUIRE(workspace && workspace_bytes >= need,
             "redundancy_raw: workspace of %lld bytes required", (long long)need);
  ZP_REQUIRE(((uintptr_t)workspace % 16) == 0, "redundancy_raw: workspace must be 16-byte aligned");
  GramArgs a;
  a.k = (const char*)k_cache; a.table = block_table;
  a.r_out = red_out;   // 16-bit caches: the row sums go here before the softmax
  a.ws_sum = (float*)workspace; a.ws_col = (int32_t*)workspace + n; a.ws_val = (float*)workspace + 2 * n;
  a.ws_chunk = (float*)workspace + 3 * n;
  a.B = B; a.NB = NB; a.BS = BS; a.Hkv = Hkv; a.D = D; a.num_pages = num_pages;
  a.k_sl = k_sl; a.k_sp = k_sp; a.threshold = threshold; a.eps = 1e-6f;
  hipStream_t st = (hipStream_t)stream;
  ZP_DISPATCH_DTYPE(dtype, {
    rc = launch_gram<T, true>(a, L, st);
    if (rc != ZP_OK) return rc;
    rc = launch_softmax<T, true>(red_out, logits_out, block_table, a.ws_sum, a.ws_col, a.ws_val, L,
                                 B, NB, BS, Hkv, num_pages, temperature, st, T::bytes == 2,
                                 (T::bytes == 4 && raw_f32_symmetric(NB, BS)) ? a.ws_chunk : nullptr);
  });
  return rc;
}
