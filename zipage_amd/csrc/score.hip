// Ragged attention scorer: softmax(window queries x paged keys), max over the GQA group,
// mean (or max) over the window, MFMA for the QK^T contraction.  The (Hq, W, T) logits the
// reference materialises are never written (unless the caller asks for them).  Rounding points
// follow the reference (logits, logit - max, softmax output and the window mean are each rounded
// to the cache dtype), so bf16/fp16 results agree with it to the last bit except where fp32
// accumulation order moves a value across a rounding boundary.
//
// Three kernels:
//   score_resident_kernel  16-bit caches, at most 2560 tokens per sequence, no logits requested:
//       ONE sweep over K.  A workgroup is one block of 32 query rows of a (layer, sequence, head);
//       its rounded logits stay in registers (two per word) and the row maximum, the row sum and
//       the output come from the registers.  Described above the kernel.
//   score_resident_f32_kernel  the same for fp32 caches: blocks of 16 query rows, one fp32 logit
//       per register, v_mfma_f32_16x16x4_f32.  Described above the kernel.
//   score_kernel           everything else (longer sequences, logits, no scratch):
//       one workgroup per (layer, sequence, kv head).  The softmax normaliser spans the whole
//       sequence, so it makes three passes over the sequence's pages, recomputing QK^T each time:
//         pass 1  row maximum of the (rounded) logits,
//         pass 2  row sum of exp(rounded(logit - max)),
//         pass 3  p = exp(.) / sum, max over the group, sum over the window, store (the group
//                 maximum is taken on the exponents x*log2(e) - log2(sum), one exponential per
//                 group).
//       fp32 caches take passes 1 and 2 in one sweep.  K tiles are staged through double-buffered
//       LDS; passes 2 and 3 re-read K from L2 / Infinity Cache.
//
// MFMA tiling (wave64, 32x32 tiles), score_kernel and score_resident_kernel: the A operand is a block of 32 query rows, row
// m = w*Gp + g (Gp = GQA group padded to a power of two), held in registers; the B operand is 32
// tokens of K read from LDS.  In the 32x32 accumulator layout a lane owns one token column and
// 16 rows ((r/4)*8 + (lane/32)*4 + r%4), so with this row order the group maximum is taken inside
// a lane (plus one cross-half exchange when Gp >= 8) and the window sum is a lane-local sum plus
// one cross-half step; the row blocks' shares meet in LDS (score_kernel: wave v owns row block v,
// tiles of 128 or 64 tokens are shared by all waves) or in the scratch (score_resident_kernel).
#include "common.h"
#include <math.h>
#include <type_traits>

namespace {

constexpr int kWaves = 4;               // waves per workgroup
constexpr int kTN16 = 32 * kWaves;      // tokens per K tile for 16-bit caches
constexpr int kOcc16 = 2;               // workgroups per CU the 16-bit kernel is compiled for
constexpr int kThreads = kWaves * 64;
constexpr int kRowWaves = 4;   // most waves along the query-row axis; the other factor splits tokens.
                               // Fewer row blocks (small window x group) use 2 or 1 row waves so
                               // that no wave idles: ScoreArgs::RW.
constexpr int kDmax = 128;
constexpr float kRefSpan = 60.f;   // exp(60) * 2^16 tokens stays far inside the fp32 range

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

template <typename T> struct Mma;
template <> struct Mma<BF16> {
  typedef bf16x8_t Frag;
  static constexpr int KPI = 16, EPL = 8, KS = kDmax / KPI, TN = kTN16, ROWB = kDmax * 2 + 16;
  __device__ static __forceinline__ f32x16_t mma(Frag a, Frag b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mma<F16> {
  typedef f16x8_t Frag;
  static constexpr int KPI = 16, EPL = 8, KS = kDmax / KPI, TN = kTN16, ROWB = kDmax * 2 + 16;
  __device__ static __forceinline__ f32x16_t mma(Frag a, Frag b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mma<F32> {
  typedef float Frag;
  static constexpr int KPI = 2, EPL = 1, KS = kDmax / KPI, TN = 16 * kWaves, ROWB = kDmax * 4 + 16;
  __device__ static __forceinline__ f32x16_t mma(Frag a, Frag b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};

struct ScoreArgs {
  const char* k;
  const char* q;
  const int32_t* seq_idx;
  const int32_t* table;
  void* out;
  void* logits;   // optional (L,B,Hq,W,NB,BS)
  float* ws;      // fp32 (L*B*Hkv, NB*BS) partial window sums, only when row rounds > 1
  int L, B, NB, BS, Hkv, Hq, G, Gp, D, W, num_pages, max_seqs;
  int64_t k_sl, k_sp, q_sl, q_ss;  // element strides
  float scale;
  int reduce_max;
  int RB;  // row blocks of 32
  int gs;  // log2(Gp)
  int RW;  // waves along the row axis: 1, 2 or 4
  float* part;    // register-resident kernel: fp32 window partials (L*B*Hkv, RB, NB*BS)
  int n_items;    // L*B*Hkv
};

template <typename T>
__device__ __forceinline__ void zero_frag(typename Mma<T>::Frag& f) {
  __builtin_memset(&f, 0, sizeof(f));
}

// Round two fp32 values to the cache dtype and back, in place.  bf16 uses the packed
// hardware conversion (one instruction for the pair).
template <typename T> struct Rnd;
template <> struct Rnd<F32> {
  __device__ static __forceinline__ void pair(float&, float&) {}
};
template <> struct Rnd<BF16> {
  __device__ static __forceinline__ void pair(float& a, float& b) {
    // v_cvt_pk_bf16_f32 with a zero in the low half: the 32-bit result IS the rounded value as
    // fp32, so each value costs one instruction and nothing has to be unpacked
    typedef __attribute__((ext_vector_type(2))) float f2;
    typedef __attribute__((ext_vector_type(2))) __bf16 b2;
    const f2 va = {0.f, a}, vb = {0.f, b};
    a = __builtin_bit_cast(float, __builtin_convertvector(va, b2));
    b = __builtin_bit_cast(float, __builtin_convertvector(vb, b2));
  }
};
template <> struct Rnd<F16> {
  __device__ static __forceinline__ void pair(float& a, float& b) {
    a = (float)(_Float16)a;
    b = (float)(_Float16)b;
  }
};

// One v_max_f32, nothing else: fmaxf() makes the compiler quiet possible signalling NaNs first
// (an extra v_max x,x per operand that is not known to be canonical, e.g. anything unpacked from
// bf16 bits), which doubles or triples the cost of the max-heavy epilogues.  No NaN occurs here.
__device__ __forceinline__ float vmax(float a, float b) {
  float d;
  asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ float vmax3(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}
__device__ __forceinline__ float vmax4(float a, float b, float c, float d) { return vmax(vmax3(a, b, c), d); }
__device__ __forceinline__ float vmax_neg(float a, float b) {  // max(a, -b)
  float d;
  asm("v_max_f32 %0, %1, -%2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}

// exp of a non-positive argument, natural base, via the hardware base-2 exponential.
__device__ __forceinline__ float exp_neg(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f);
}

// 2^y through the hardware exponential (y <= 0 here; -inf gives 0).
__device__ __forceinline__ float exp2_hw(float y) {
  return __builtin_amdgcn_exp2f(y);
}

// GPC: padded GQA group size known at compile time (0: read it from the arguments); RMAXC: window
// reduction known at compile time (0 mean, 1 max, -1: from the arguments).  The common shape
// (group 4, mean) gets its own instantiation: straight-line epilogues instead of uniform branches
// and compute-both-then-select.
template <typename T, bool LOGITS, int GPC, int RMAXC>
__global__ __launch_bounds__(kThreads, (T::bytes == 2 ? kOcc16 : 1)) void score_kernel(ScoreArgs p) {
  typedef Mma<T> M;
  const int GpV = GPC > 0 ? GPC : p.Gp;
  const int gsV = GPC == 8 ? 3 : GPC == 4 ? 2 : GPC == 2 ? 1 : p.gs;
  const bool rmaxV = RMAXC >= 0 ? (RMAXC != 0) : (p.reduce_max != 0);
  typedef typename M::Frag Frag;
  constexpr int TN = M::TN, ROWB = M::ROWB, KS = M::KS;
  const int RW = p.RW, TW = kWaves / RW;  // row waves x token waves
  const int NSUB = TN / 32 / TW;          // subtiles per wave and tile
  constexpr int PIECES = kDmax * T::bytes / 16;       // 16-byte pieces per full key row
  constexpr int ROWS_PER_IT = kThreads / PIECES;      // rows staged per iteration
  constexpr int STAGE_IT = TN / ROWS_PER_IT;          // iterations (== 8)

  extern __shared__ __align__(16) char smem[];
  char* kbuf0 = smem;
  char* kbuf1 = smem + TN * ROWB;
  float* part = (float*)(smem + 2 * TN * ROWB);        // [2][kRowWaves][TN]
  float* stat = part + 2 * kRowWaves * TN;              // [kWaves][32] row statistics
  int2* vinfo = (int2*)(stat + kWaves * 32);           // [NB] valid pages: (page id, index in the table | last << 30)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int rbw = wave % RW, tg = wave / RW;  // row-block wave, token group
  const int h = blockIdx.x % p.Hkv;
  const int b = (blockIdx.x / p.Hkv) % p.B;
  const int l = blockIdx.x / (p.Hkv * p.B);
  const int Tn = p.NB * p.BS;
  const int64_t orow = (((int64_t)l * p.B + b) * p.Hkv + h);

  // ---- valid page list (block-uniform), zero pad-page outputs
  __shared__ int nvalid_s;
  if (p.NB <= 64) {
    // one lane per table entry; a ballot packs the usable pages in table order
    if (wave == 0) {
      const int code = lane < p.NB ? p.table[(int64_t)b * p.NB + lane] : -1;
      const int pid = page_is_pad(code) ? -1 : page_id(code);
      const bool ok = pid >= 0 && pid < p.num_pages;
      const unsigned long long okm = __builtin_amdgcn_ballot_w64(ok);
      if (ok) {
        const int n = __builtin_popcountll(okm & lanemask_lt());
        vinfo[n] = make_int2(pid, lane | (page_is_last(code) ? (1 << 30) : 0));
      }
      if (lane == 0) nvalid_s = __builtin_popcountll(okm);
    }
  } else if (tid == 0) {
    int n = 0;
    for (int j = 0; j < p.NB; ++j) {
      const int code = p.table[(int64_t)b * p.NB + j];
      const int pid = page_is_pad(code) ? -1 : page_id(code);
      if (pid >= 0 && pid < p.num_pages) {
        vinfo[n] = make_int2(pid, j | (page_is_last(code) ? (1 << 30) : 0));
        ++n;
      }
    }
    nvalid_s = n;
  }
  // with a head dim below 128 the tail of every LDS row must read as zero
  if (p.D * T::bytes < kDmax * T::bytes)
    for (int i = tid; i < 2 * TN * ROWB / 4; i += kThreads) ((uint32_t*)smem)[i] = 0u;
  __syncthreads();
  const int nvalid = nvalid_s;
  {
    // pad pages (and unusable ids) score exactly 0; their logits stay -inf
    for (int j = 0; j < p.NB; ++j) {
      const int code = p.table[(int64_t)b * p.NB + j];
      const int pid = page_is_pad(code) ? -1 : page_id(code);
      if (pid >= 0 && pid < p.num_pages) continue;
      for (int s = tid; s < p.BS; s += kThreads)
        Elem<T>::st(p.out, orow * Tn + (int64_t)j * p.BS + s, 0.f);
    }
  }
  int seq = p.seq_idx[b];
  const bool seq_ok = seq >= 0 && seq < p.max_seqs;
  if (!seq_ok) seq = 0;

  const int tiles_per_page = p.BS / TN;
  const int ntiles = nvalid * tiles_per_page;
  // tile -> (valid page, token offset); a shift when a page holds a power-of-two number of tiles
  const int tpp_shift = (tiles_per_page & (tiles_per_page - 1)) == 0 ? __builtin_ctz(tiles_per_page) : -1;
  auto tile_page = [&](int tile) { return tpp_shift >= 0 ? tile >> tpp_shift : tile / tiles_per_page; };
  const int dpieces = p.D * T::bytes / 16;  // valid 16-byte pieces per key row
  const int64_t k_row = (int64_t)p.Hkv * p.D * T::bytes;
  const char* kbase = p.k + (l * p.k_sl) * T::bytes + (int64_t)h * p.D * T::bytes;

  // staging coordinates of this thread; the byte offsets of its eight pieces inside a tile are
  // kept as 32-bit registers and the tile base is wave-uniform, so a load needs no address math
  const int st_piece = tid % PIECES, st_row0 = tid / PIECES;
  vec16 pre[STAGE_IT];
  uint32_t ld_off[STAGE_IT];
#pragma unroll
  for (int i = 0; i < STAGE_IT; ++i)
    ld_off[i] = (uint32_t)((st_row0 + i * ROWS_PER_IT) * k_row + st_piece * 16);

  auto issue_loads = [&](int tile, int pid) {
    const int vp = tile_page(tile), toff = (tile - vp * tiles_per_page) * TN;
    const char* src = kbase + (int64_t)pid * p.k_sp * T::bytes + (int64_t)toff * k_row;
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      if (st_piece < dpieces) pre[i] = *(const vec16*)(src + ld_off[i]);
    }
  };
  auto commit_loads = [&](char* buf) {
#pragma unroll
    for (int i = 0; i < STAGE_IT; ++i) {
      const int row = st_row0 + i * ROWS_PER_IT;
      if (st_piece < dpieces) {
        uint2* d = (uint2*)(buf + row * ROWB + st_piece * 16);
        d[0] = make_uint2(pre[i].x, pre[i].y);
        d[1] = make_uint2(pre[i].z, pre[i].w);
      }
    }
  };

  const int NR = (p.RB + RW - 1) / RW;  // row rounds
  const float ascale = fabsf(p.scale);
  const float sgn = p.scale < 0.f ? -1.f : 1.f;
  for (int rr = 0; rr < NR; ++rr) {
    const int rb = rr * RW + rbw;
    const bool active = rb < p.RB;
    // ---- A fragments: query rows of this wave's row block
    Frag afrag[KS];
    const int mrow = rb * 32 + col;                 // row this lane loads
    const int a_w = mrow >> gsV, a_g = mrow & (GpV - 1);
    const bool a_ok = active && seq_ok && a_w < p.W && a_g < p.G;
    {
      const char* qrow = p.q + ((int64_t)l * p.q_sl + (int64_t)seq * p.q_ss +
                                ((int64_t)a_w * p.Hq + (int64_t)h * p.G + a_g) * p.D) * T::bytes;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        // fp32: the order of the contraction index is free as long as both operands agree;
        // k-step 4j + i of wave half `half` takes element 8j + 4 half + i, so that a lane's B
        // operands for four steps are one 16-byte LDS read
        const int k0 = T::bytes == 4 ? 8 * (s >> 2) + 4 * half + (s & 3) : s * M::KPI + half * M::EPL;
        if (a_ok && k0 < p.D) afrag[s] = *(const Frag*)(qrow + (int64_t)k0 * T::bytes);
        else zero_frag<T>(afrag[s]);
      }
    }
    // the query fragments are complete before the tile loop starts, so waits inside it only
    // concern that loop's own loads
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(afrag[s]));
    // rows owned by this lane in the accumulator layout: (r/4)*8 + half*4 + r%4
    const int row0 = rb * 32 + half * 4;
    float cl[16], mx[16];   // cl = -log2(row sum): p = 2^(x*log2(e) + cl)
#pragma unroll
    for (int r = 0; r < 16; ++r) { mx[r] = 0.f; cl[r] = -INFINITY; }
    // fp32 caches only (PASS 3): this lane's reference logit and running maximum per row
    float ref[T::bytes == 4 ? 16 : 1], mrun[T::bytes == 4 ? 16 : 1];
    bool far_off = false;   // PASS 3: a logit more than kRefSpan above its lane's reference

    // One sweep over the sequence's K tiles.  PASS 0: row max; 1: row sum of exp; 2: output;
    // 3 (fp32 caches): row max AND row sum in one sweep.  Without roundings to a 16-bit dtype the
    // softmax does not depend on which finite reference is subtracted before the exponential, so
    // every lane sums exp(s - ref) against its own first logit of the row, tracks its maximum,
    // and the lanes' sums are brought to the common maximum afterwards:
    // sum_t exp(s_t - m) = sum_lanes exp(ref_lane - m) sum_{t in lane} exp(s_t - ref_lane).
    // Exact as long as no logit lies more than kRefSpan above its lane's reference (fp32 range);
    // otherwise the caller falls back to the two separate sweeps.
    auto sweep = [&](auto pass_c) {
      constexpr int PASS = decltype(pass_c)::value;
      auto finish_tile = [&](int tile, int j, int toff) {
        if (tid < TN) {
          const float* pt = part + (tile & 1) * kRowWaves * TN;
          float v = pt[tid];
#pragma unroll
          for (int w2 = 1; w2 < RW; ++w2)
            v = rmaxV ? fmaxf(v, pt[w2 * TN + tid]) : v + pt[w2 * TN + tid];
          const int64_t oi = orow * Tn + (int64_t)j * p.BS + toff + tid;
          if (NR > 1) {
            float* wsp = p.ws + oi;
            if (rr > 0) v = rmaxV ? fmaxf(v, *wsp) : v + *wsp;
            if (rr + 1 < NR) *wsp = v;
          }
          if (rr + 1 == NR)
            Elem<T>::st(p.out, oi, rmaxV ? v : Elem<T>::rnd(v / (float)p.W));
        }
      };
      float run[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) run[r] = PASS == 0 ? -INFINITY : 0.f;
      if constexpr (PASS == 3) {
#pragma unroll
        for (int r = 0; r < 16; ++r) { mrun[r] = -INFINITY; ref[r] = 0.f; }
      }
      // The middle sweep walks the tiles backwards: it starts on the tiles the first sweep read
      // last (still in L2) and ends on those the third sweep reads first.
      auto order = [&](int i) { return PASS == 1 ? ntiles - 1 - i : i; };
      // (page id, slot) of a tile; the entry of tile it+2 is requested a whole tile before its
      // page id is needed, so the tile loop never waits for this LDS read
      auto tile_info = [&](int i) { return vinfo[tile_page(order(i < ntiles ? i : ntiles - 1))]; };
      int vs = 0;          // slot word of the current tile
      int2 info_next = make_int2(0, 0);   // entry of tile it+1
      if (ntiles > 0) {
        const int2 i0 = tile_info(0);
        vs = __builtin_amdgcn_readfirstlane(i0.y);
        issue_loads(order(0), __builtin_amdgcn_readfirstlane(i0.x));
        info_next = tile_info(1);
        commit_loads(kbuf0);
      }
      __syncthreads();
      for (int it = 0; it < ntiles; ++it) {
        const int tile = order(it);
        char* cur = (it & 1) ? kbuf1 : kbuf0;
        char* nxt = (it & 1) ? kbuf0 : kbuf1;
        const int pid_next = __builtin_amdgcn_readfirstlane(info_next.x);
        const int vs_next = __builtin_amdgcn_readfirstlane(info_next.y);
        info_next = tile_info(it + 2);
        if (it + 1 < ntiles) issue_loads(order(it + 1), pid_next);
        const int vp = tile_page(tile), toff = (tile - vp * tiles_per_page) * TN;
        const int j = vs & 0xffff;
        const bool last = (vs >> 30) & 1;
        if (active) {
          int sti = 0;
          if constexpr (PASS == 0 && !LOGITS && T::bytes == 2) {
            // The max sweep has little to do per product, so a lone chain of eight dependent MFMAs
            // behind an LDS round trip leaves the matrix core idle half of the time: two subtiles
            // are multiplied at once, their MFMAs alternating between two accumulators.
#pragma unroll 1
            for (; sti + 1 < NSUB; sti += 2) {
              const int st = tg * NSUB + sti;
              const char* browA = cur + (st * 32 + col) * ROWB + half * M::EPL * T::bytes;
              const char* browB = browA + 32 * ROWB;
              f32x16_t accA, accB;
#pragma unroll
              for (int r = 0; r < 16; ++r) { accA[r] = 0.f; accB[r] = 0.f; }
              constexpr int KH = KS / 2;
#pragma unroll
              for (int s0 = 0; s0 < KS; s0 += KH) {
                Frag bA[KH], bB[KH];
#pragma unroll
                for (int s = 0; s < KH; ++s) bA[s] = *(const Frag*)(browA + (s0 + s) * M::KPI * T::bytes);
#pragma unroll
                for (int s = 0; s < KH; ++s) bB[s] = *(const Frag*)(browB + (s0 + s) * M::KPI * T::bytes);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < KH; ++s) {
                  accA = M::mma(afrag[s0 + s], bA[s], accA);
                  accB = M::mma(afrag[s0 + s], bB[s], accB);
                }
              }
              if (last && (toff + st * 32 + 63 > p.BS - p.W)) {
                const int slotA = toff + st * 32 + col;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                  const int w = (row0 + (r >> 2) * 8 + (r & 3)) >> gsV;
                  if (slotA > p.BS - p.W + w) accA[r] = -sgn * INFINITY;
                  if (slotA + 32 > p.BS - p.W + w) accB[r] = -sgn * INFINITY;
                }
              }
              if (sgn > 0.f) {
#pragma unroll
                for (int r = 0; r < 16; ++r) run[r] = vmax3(run[r], accA[r], accB[r]);
              } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) run[r] = vmax_neg(vmax_neg(run[r], accA[r]), accB[r]);
              }
            }
          }
          // one 32 x 32 block of products: query row block x the tokens of subtile st
          auto products = [&](int st) {
            f32x16_t acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
            const char* brow = cur + (st * 32 + col) * ROWB + half * M::EPL * T::bytes;
            const char* brow4 = cur + (st * 32 + col) * ROWB + half * 16;   // fp32 operand order
            // all B fragments of the subtile are requested before the first MFMA needs one
            constexpr int KB = KS < 8 ? KS : 8;
#pragma unroll
            for (int s0 = 0; s0 < KS; s0 += KB) {
              Frag bfr[KB];
#pragma unroll
              for (int s = 0; s < KB; ++s) {
                if constexpr (T::bytes == 4) {
                  if ((s & 3) == 0) {
                    const float4 b4 = *(const float4*)(brow4 + ((s0 + s) >> 2) * 32);
                    __builtin_memcpy(&bfr[s], &b4, 16);
                  }
                } else {
                  bfr[s] = *(const Frag*)(brow + (s0 + s) * M::KPI * T::bytes);
                }
              }
              __builtin_amdgcn_sched_barrier(0);  // keep the reads grouped ahead of the MFMAs
#pragma unroll
              for (int s = 0; s < KB; ++s) acc = M::mma(afrag[s0 + s], bfr[s], acc);
            }
            return acc;
          };
          // what a sweep does with a block of products.  MASKED: the causal mask of a last page
          // may apply (a uniform branch; the unmasked form is a single basic block)
          auto epilogue = [&](f32x16_t acc, int st, int sti, auto masked_c) {
            constexpr bool MASKED = decltype(masked_c)::value;
            const int slot = toff + st * 32 + col;  // token slot inside its page
            // causal mask: only the tail of the last page can be hidden from a window row
            if (MASKED && last && (toff + st * 32 + 31 > p.BS - p.W)) {
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int w = (row0 + (r >> 2) * 8 + (r & 3)) >> gsV;
                if (slot > p.BS - p.W + w) acc[r] = -sgn * INFINITY;
              }
            }
            if constexpr (PASS == 3) {
              const bool first = it == 0 && sti == 0;   // uniform
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const float sv = acc[r] * p.scale;      // masked entries: -inf
                if (first) ref[r] = sv > -INFINITY ? sv : 0.f;
                mrun[r] = vmax(mrun[r], sv);
                run[r] += exp2_hw((sv - ref[r]) * 1.44269504088896340736f);
              }
            } else if constexpr (PASS == 0) {
              // max of sign(scale)*acc; scaling is monotone, so it is applied once at the end
              if (sgn > 0.f) {  // block-uniform: the negation is a free source modifier
#pragma unroll
                for (int r = 0; r < 16; ++r) run[r] = vmax(run[r], acc[r]);
              } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) run[r] = vmax_neg(run[r], acc[r]);
              }
              if constexpr (LOGITS) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                  const int m = row0 + (r >> 2) * 8 + (r & 3);
                  const int w = m >> gsV, g = m & (GpV - 1);
                  if (w < p.W && g < p.G) {
                    const int64_t li =
                        ((((int64_t)l * p.B + b) * p.Hq + (int64_t)h * p.G + g) * p.W + w) * Tn +
                        (int64_t)j * p.BS + slot;
                    Elem<T>::st(p.logits, li, acc[r] * p.scale);
                  }
                }
              }
            } else {
              float pv[16];
#pragma unroll
              for (int r = 0; r < 16; r += 2) {
                float s0 = acc[r] * p.scale, s1 = acc[r + 1] * p.scale;
                Rnd<T>::pair(s0, s1);
                float x0 = s0 - mx[r], x1 = s1 - mx[r + 1];
                Rnd<T>::pair(x0, x1);
                if constexpr (PASS == 1) {
                  run[r] += exp_neg(x0);
                  run[r + 1] += exp_neg(x1);
                } else {
                  // p = exp(x) / sum = 2^(x*log2(e) - log2(sum)).  The exponential and the rounding
                  // to the cache dtype are monotone, so the maximum over the group is taken on the
                  // exponents and a group of n rows costs one exponential and one rounding
                  pv[r] = __builtin_fmaf(x0, 1.44269504088896340736f, cl[r]);
                  pv[r + 1] = __builtin_fmaf(x1, 1.44269504088896340736f, cl[r + 1]);
                }
              }
              if constexpr (PASS == 2) {
                // group max inside the lane, then window sum / max
                float red;
                const int Gp = GpV;
                if (Gp < 2) {  // no group: every probability is rounded on its own
#pragma unroll
                  for (int r = 0; r < 16; r += 2) {
                    pv[r] = exp2_hw(pv[r]);
                    pv[r + 1] = exp2_hw(pv[r + 1]);
                    Rnd<T>::pair(pv[r], pv[r + 1]);
                  }
                }
                if (Gp >= 4) {
                  float q4[4];
#pragma unroll
                  for (int q = 0; q < 4; ++q)
                    q4[q] = vmax4(pv[4 * q], pv[4 * q + 1], pv[4 * q + 2], pv[4 * q + 3]);
                  if (Gp >= 8) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) q4[q] = vmax(q4[q], lane_xor32(q4[q]));
                  }
                  if (Gp < 16) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) q4[q] = exp2_hw(q4[q]);
                    Rnd<T>::pair(q4[0], q4[1]);
                    Rnd<T>::pair(q4[2], q4[3]);
                  }
                  if (Gp >= 16) {
                    q4[0] = vmax(q4[0], q4[1]);
                    q4[2] = vmax(q4[2], q4[3]);
                    if (Gp >= 32) {
                      red = exp2_hw(vmax(q4[0], q4[2]));
                      float dummy = red;
                      Rnd<T>::pair(red, dummy);
                    } else {
                      q4[0] = exp2_hw(q4[0]);
                      q4[2] = exp2_hw(q4[2]);
                      Rnd<T>::pair(q4[0], q4[2]);
                      red = rmaxV ? vmax(q4[0], q4[2]) : q4[0] + q4[2];
                    }
                  } else {
                    red = rmaxV ? vmax4(q4[0], q4[1], q4[2], q4[3])
                                       : (q4[0] + q4[1]) + (q4[2] + q4[3]);
                  }
                } else {
                  float t8[8];
                  if (Gp == 2) {
#pragma unroll
                    for (int q = 0; q < 8; ++q) t8[q] = exp2_hw(vmax(pv[2 * q], pv[2 * q + 1]));
#pragma unroll
                    for (int q = 0; q < 8; q += 2) Rnd<T>::pair(t8[q], t8[q + 1]);
                  } else {
#pragma unroll
                    for (int q = 0; q < 8; ++q)
                      t8[q] = rmaxV ? vmax(pv[2 * q], pv[2 * q + 1]) : pv[2 * q] + pv[2 * q + 1];
                  }
                  if (rmaxV) {
                    red = vmax3(vmax3(t8[0], t8[1], t8[2]), vmax3(t8[3], t8[4], t8[5]), vmax(t8[6], t8[7]));
                  } else {
                    red = ((t8[0] + t8[1]) + (t8[2] + t8[3])) + ((t8[4] + t8[5]) + (t8[6] + t8[7]));
                  }
                }
                if (Gp < 8) {  // the two lane halves hold different windows
                  const float o = lane_xor32(red);
                  red = rmaxV ? vmax(red, o) : red + o;
                }
                if (half == 0) part[((tile & 1) * kRowWaves + rbw) * TN + st * 32 + col] = red;
              }
            }
                    };
          if constexpr ((PASS == 1 || PASS == 2) && !LOGITS && T::bytes == 2) {
            // Sum and output sweeps, whole tiles away from the causal mask: the products of subtile
            // k+1 are issued between the epilogue instructions of subtile k, so the matrix core
            // works while the vector unit runs the epilogue (a lone wave would do one after the other).
            if (NSUB == 4 && !last) {
              const int st0 = tg * 4;
              auto interleave = [&]() {
                __builtin_amdgcn_sched_group_barrier(0x100, KS, 0);     // the LDS reads first
#pragma unroll
                for (int s = 0; s < KS; ++s) {
                  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);    // one MFMA
                  __builtin_amdgcn_sched_group_barrier(0x002, PASS == 1 ? 14 : 13, 0);   // a share of the epilogue
                }
              };
              const std::false_type unmasked{};
              const f32x16_t a0 = products(st0);
              __builtin_amdgcn_sched_barrier(0);
              const f32x16_t a1 = products(st0 + 1);
              epilogue(a0, st0, 0, unmasked);
              interleave();
              __builtin_amdgcn_sched_barrier(0);
              const f32x16_t a2 = products(st0 + 2);
              epilogue(a1, st0 + 1, 1, unmasked);
              interleave();
              __builtin_amdgcn_sched_barrier(0);
              const f32x16_t a3 = products(st0 + 3);
              epilogue(a2, st0 + 2, 2, unmasked);
              interleave();
              __builtin_amdgcn_sched_barrier(0);
              epilogue(a3, st0 + 3, 3, unmasked);
              sti = NSUB;
            }
          }
#pragma unroll 1
          for (; sti < NSUB; ++sti) {
            const int st = tg * NSUB + sti;
            epilogue(products(st), st, sti, std::true_type{});
          }
        } else if (PASS == 2) {
#pragma unroll
          for (int sti = 0; sti < NSUB; ++sti)
            if (half == 0) part[((tile & 1) * kRowWaves + rbw) * TN + (tg * NSUB + sti) * 32 + col] = 0.f;
        }
        if (it + 1 < ntiles) commit_loads(nxt);
        __syncthreads();
        // the window partials of this tile are complete: combine the waves' shares while the
        // next tile is being computed (the buffer is rewritten two tiles later)
        if constexpr (PASS == 2) finish_tile(tile, j, toff);
        vs = vs_next;
      }
      // the xor butterfly leaves the row result in all 32 lanes that share the row; the
      // token-group waves that share a row block then combine their halves through LDS
      if constexpr (PASS == 3) {
        // row maximum over the 32 lanes of the row and the token-group waves, then the lanes' sums
        // at that maximum
        float mrow[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          far_off |= mrun[r] - ref[r] > kRefSpan;
          const float v = half_max(mrun[r]);
          mrow[r] = v;
          if (col == 0) stat[wave * 32 + (r >> 2) * 8 + half * 4 + (r & 3)] = v;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = mrow[r];
#pragma unroll
          for (int g2 = 1; g2 < TW; ++g2) {
            const int ow = ((tg + g2) % TW) * RW + rbw;
            v = fmaxf(v, stat[ow * 32 + (r >> 2) * 8 + half * 4 + (r & 3)]);
          }
          mx[r] = v;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          // a lane that saw only masked tokens has run == 0 and contributes nothing
          const float t = run[r] * exp2_hw((ref[r] - mx[r]) * 1.44269504088896340736f);
          const float v = half_sum(run[r] > 0.f ? t : 0.f);
          run[r] = v;
          if (col == 0) stat[wave * 32 + (r >> 2) * 8 + half * 4 + (r & 3)] = v;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = run[r];
#pragma unroll
          for (int g2 = 1; g2 < TW; ++g2) {
            const int ow = ((tg + g2) % TW) * RW + rbw;
            v += stat[ow * 32 + (r >> 2) * 8 + half * 4 + (r & 3)];
          }
          const int m = row0 + (r >> 2) * 8 + (r & 3);
          const bool ok = active && (m >> gsV) < p.W && (m & (GpV - 1)) < p.G;
          cl[r] = ok ? -__builtin_amdgcn_logf(v) : -INFINITY;
        }
        __syncthreads();
      } else if constexpr (PASS < 2) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float v = PASS == 0 ? half_max(run[r]) : half_sum(run[r]);
          run[r] = v;
          if (col == 0) stat[wave * 32 + (r >> 2) * 8 + half * 4 + (r & 3)] = v;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = run[r];
#pragma unroll
          for (int g2 = 1; g2 < TW; ++g2) {
            const int ow = ((tg + g2) % TW) * RW + rbw;
            const float t = stat[ow * 32 + (r >> 2) * 8 + half * 4 + (r & 3)];
            v = PASS == 0 ? fmaxf(v, t) : v + t;
          }
          if constexpr (PASS == 0) {
            mx[r] = Elem<T>::rnd(v * ascale);
          } else {
            const int m = row0 + (r >> 2) * 8 + (r & 3);
            const bool ok = active && (m >> gsV) < p.W && (m & (GpV - 1)) < p.G;
            cl[r] = ok ? -__builtin_amdgcn_logf(v) : -INFINITY;   // rows outside the window or group never win a maximum
          }
        }
        __syncthreads();
      }
    };
    bool merged = false;
    if constexpr (T::bytes == 4 && !LOGITS) {
      sweep(std::integral_constant<int, 3>{});
      merged = !__syncthreads_or(far_off ? 1 : 0);
    }
    if (!merged) {
      sweep(std::integral_constant<int, 0>{});
      sweep(std::integral_constant<int, 1>{});
    }
    sweep(std::integral_constant<int, 2>{});
  }
}


// ================================================================ register-resident scorer
// For 16-bit caches and sequences of at most kResTiles x 128 tokens the three sweeps collapse into
// ONE sweep over K: the rounded logits of a block of 32 query rows stay in registers, two per
// 32-bit word, and the row maximum, the row sum and the output are computed from the registers.
//
// A workgroup is one (layer, sequence, kv head, block of 32 query rows) unit; its four waves split
// the tokens: wave t owns tokens [128 i + 32 t, 128 i + 32 t + 32) of every 128-token tile i, i.e.
// 8 words per tile and lane.  Every wave streams its own 32-row K blocks from global memory
// straight into LDS (no staging registers, no workgroup barrier in the sweep) two blocks ahead.
// The row maxima and sums of the four waves meet in LDS (two barriers per unit).  The window
// reduction of a unit covers only its own windows, so a unit writes fp32 partial sums and
// score_combine_kernel adds the units of a (layer, sequence, head) in a fixed order, divides by
// the window length and rounds -- the same arithmetic, in the same order, as the three-sweep
// kernel's combine across its row-block waves.
//
// LDS layout of a 32-row block (rows of 256 bytes = 16 pieces of 16 bytes): a load instruction
// fills 1 KB of consecutive LDS with four rows, so padding can only go between groups of four rows.
// Inside a group piece g of row r sits at (g / 4) * 256 + r * 64 + (g % 4) * 16 and groups are
// 1040 bytes apart: the sixteen lanes that read the same piece of sixteen consecutive rows then
// fall into sixteen different 16-byte bank groups, a quad of lanes still fetches 64 consecutive
// bytes of one row, and the fragment of contraction step s is an immediate offset from one base.
constexpr int kResTiles = 20;
constexpr int kGrp = 1040;
constexpr int kSubBytes = 8 * kGrp;

template <typename T> struct Pack2;
template <> struct Pack2<BF16> {
  __device__ static __forceinline__ uint32_t pack(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float f2;
    typedef __attribute__((ext_vector_type(2))) __bf16 b2;
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, b2));
  }
  __device__ static __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  __device__ static __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
};
template <> struct Pack2<F16> {
  typedef __attribute__((ext_vector_type(2))) _Float16 h2;
  __device__ static __forceinline__ uint32_t pack(float lo, float hi) {
    const h2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  __device__ static __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(h2, w)[0]; }
  __device__ static __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(h2, w)[1]; }
};

// Group maximum and window reduction of the sixteen exponents a lane holds for one token
// (pv[r] = x log2(e) - log2(row sum), rows (r/4)*8 + half*4 + r%4 of the block): the probability
// is 2^pv rounded to the cache dtype; exponential and rounding are monotone, so the maximum over
// the group is taken first.  Returns the lane's share of the window sum (or maximum) over the
// windows of the block, both wave halves already combined when they hold different windows.
template <typename T>
__device__ __forceinline__ float group_window_reduce(float (&pv)[16], int Gp, bool rmaxV) {
  float red;
  if (Gp < 2) {
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      pv[r] = exp2_hw(pv[r]);
      pv[r + 1] = exp2_hw(pv[r + 1]);
      Rnd<T>::pair(pv[r], pv[r + 1]);
    }
  }
  if (Gp >= 4) {
    float q4[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      q4[q] = vmax4(pv[4 * q], pv[4 * q + 1], pv[4 * q + 2], pv[4 * q + 3]);
    if (Gp >= 8) {
#pragma unroll
      for (int q = 0; q < 4; ++q) q4[q] = vmax(q4[q], lane_xor32(q4[q]));
    }
    if (Gp < 16) {
#pragma unroll
      for (int q = 0; q < 4; ++q) q4[q] = exp2_hw(q4[q]);
      Rnd<T>::pair(q4[0], q4[1]);
      Rnd<T>::pair(q4[2], q4[3]);
    }
    if (Gp >= 16) {
      q4[0] = vmax(q4[0], q4[1]);
      q4[2] = vmax(q4[2], q4[3]);
      if (Gp >= 32) {
        red = exp2_hw(vmax(q4[0], q4[2]));
        float dummy = red;
        Rnd<T>::pair(red, dummy);
      } else {
        q4[0] = exp2_hw(q4[0]);
        q4[2] = exp2_hw(q4[2]);
        Rnd<T>::pair(q4[0], q4[2]);
        red = rmaxV ? vmax(q4[0], q4[2]) : q4[0] + q4[2];
      }
    } else {
      red = rmaxV ? vmax4(q4[0], q4[1], q4[2], q4[3]) : (q4[0] + q4[1]) + (q4[2] + q4[3]);
    }
  } else {
    float t8[8];
    if (Gp == 2) {
#pragma unroll
      for (int q = 0; q < 8; ++q) t8[q] = exp2_hw(vmax(pv[2 * q], pv[2 * q + 1]));
#pragma unroll
      for (int q = 0; q < 8; q += 2) Rnd<T>::pair(t8[q], t8[q + 1]);
    } else {
#pragma unroll
      for (int q = 0; q < 8; ++q) t8[q] = rmaxV ? vmax(pv[2 * q], pv[2 * q + 1]) : pv[2 * q] + pv[2 * q + 1];
    }
    if (rmaxV) {
      red = vmax3(vmax3(t8[0], t8[1], t8[2]), vmax3(t8[3], t8[4], t8[5]), vmax(t8[6], t8[7]));
    } else {
      red = ((t8[0] + t8[1]) + (t8[2] + t8[3])) + ((t8[4] + t8[5]) + (t8[6] + t8[7]));
    }
  }
  if (Gp < 8) {  // the two lane halves hold different windows
    const float o = lane_xor32(red);
    red = rmaxV ? vmax(red, o) : red + o;
  }
  return red;
}

// TPP: 128-token tiles per page when known at compile time (0: from the arguments); with it
// the page of every unrolled tile is a constant and its id comes from a lane of a register.
template <typename T, int GPC, int RMAXC, int TPP>
__global__ __launch_bounds__(kThreads, 2) void score_resident_kernel(ScoreArgs p) {
  typedef Mma<T> M;
  typedef typename M::Frag Frag;
  typedef Pack2<T> P2;
  constexpr int KS = M::KS;   // 8 contraction steps of 16
  const int GpV = GPC > 0 ? GPC : p.Gp;
  const int gsV = GPC == 8 ? 3 : GPC == 4 ? 2 : GPC == 2 ? 1 : p.gs;
  const bool rmaxV = RMAXC >= 0 ? (RMAXC != 0) : (p.reduce_max != 0);

  extern __shared__ __align__(16) char smem[];
  float* stat = (float*)(smem + kWaves * 2 * kSubBytes);   // [kWaves][32]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, col = lane & 31;
#ifdef ZP_RES_STAMP
  // Measurement build: wave 0 of every unit records the core-clock counter at the phase
  // boundaries and the constant-rate counter at both ends, behind the window partials
  // (the caller makes the workspace 64 bytes per unit larger).
  long long stamp[8];
  int nstamp = 0;
  const long long wall0 = wall_clock64();
#define ZP_STAMP() do { stamp[nstamp++] = clock64(); } while (0)
#else
#define ZP_STAMP() do { } while (0)
#endif
  ZP_STAMP();
  // unit -> (item, row block): workgroup ids are dealt round-robin to the 8 XCDs; the row blocks
  // of an item get consecutive ids ON ONE XCD, so they run at the same time behind one L2 and
  // the item's keys leave HBM once
  const int xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
  const int rb = loc % p.RB;
  const int item = (loc / p.RB) * 8 + xcd;
  if (item >= p.n_items) return;
  const int h = item % p.Hkv;
  const int b = (item / p.Hkv) % p.B;
  const int l = item / (p.Hkv * p.B);
  const int Tn = p.NB * p.BS;

  // Every wave builds the list of usable pages for itself (no LDS, no barrier): lane j reads table
  // entry j, a ballot ranks the usable ones, and a lane permute leaves entry n of the list in lane
  // n as (page id, table index | last << 30).
  const int code = lane < p.NB ? p.table[(int64_t)b * p.NB + lane] : -1;
  int seq = p.seq_idx[b];
  int2 myinfo;
  int nvalid;
  {
    const int pid = page_is_pad(code) ? -1 : page_id(code);
    const bool ok = pid >= 0 && pid < p.num_pages;
    const unsigned long long okm = __builtin_amdgcn_ballot_w64(ok);
    nvalid = __builtin_popcountll(okm);
    const int dst = ok ? __builtin_popcountll(okm & lanemask_lt())
                       : nvalid + __builtin_popcountll(~okm & lanemask_lt());
    myinfo.x = __builtin_amdgcn_ds_permute(dst << 2, pid);
    myinfo.y = __builtin_amdgcn_ds_permute(dst << 2, lane | (page_is_last(code) ? (1 << 30) : 0));
  }
  const int dpieces = p.D * T::bytes / 16;
  char* kb = smem + wave * 2 * kSubBytes;    // this wave's two K blocks
  if (dpieces < 16) {   // the tail of every staged row must read as zero
    for (int i = lane; i < 2 * kSubBytes / 4; i += 64) ((uint32_t*)kb)[i] = 0u;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  const bool seq_ok = seq >= 0 && seq < p.max_seqs;
  if (!seq_ok) seq = 0;

  const int tiles_per_page = TPP > 0 ? TPP : p.BS / 128;
  const int ntiles = nvalid * tiles_per_page;
  auto tile_page = [&](int tile) { return tile / (TPP > 0 ? TPP : tiles_per_page); };
  auto page_word = [&](int v, int vp) {   // entry vp of the list, wave-uniform
    if constexpr (TPP > 0) return __builtin_amdgcn_readlane(v, vp);
    else return __builtin_amdgcn_readfirstlane(__builtin_amdgcn_ds_bpermute(vp << 2, v));
  };
  const int64_t k_row = (int64_t)p.Hkv * p.D * T::bytes;
  const char* kbase = p.k + (l * p.k_sl) * T::bytes + (int64_t)h * p.D * T::bytes;
  const int wtok = wave * 32;   // this wave's tokens inside a tile

  // ---- staging: a load instruction moves four rows; lane -> (row of the group, piece).  The
  // rows go through a buffer descriptor based at the block's first row, so an instruction needs
  // one fixed per-lane offset, a scalar offset and no address arithmetic.
  const int st_g = (lane >> 4) * 4 + (lane & 3), st_r = (lane >> 2) & 3;
  const int st_off = (int)(st_r * k_row + st_g * 16);
  const bool st_ok = st_g < dpieces;
  const int grp_step = (int)(4 * k_row);
  typedef void __attribute__((address_space(3))) * lptr_t;
  auto issue = [&](int tile, char* buf) {
    const int vp = tile_page(tile);
    const int pid = page_word(myinfo.x, vp);
    const int toff = (tile - vp * tiles_per_page) * 128 + wtok;
    const char* src = kbase + (int64_t)pid * p.k_sp * T::bytes + (int64_t)toff * k_row;
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, (int)(32 * k_row), 0x00020000);
    if (st_ok) {
#ifdef ZP_RES_HALFDMA   // measurement only: half of the rows are fetched, results are wrong
#define ZP_DMA_N 4
#else
#define ZP_DMA_N 8
#endif
#pragma unroll
      for (int i = 0; i < ZP_DMA_N; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(buf + i * kGrp), 16, st_off,
                                                 i * grp_step, 0, 0);
    }
  };
  // fragment of step s of this lane's row: base + (s / 2) * 256 + (s % 2) * 32
  const int rd_off = (col >> 2) * kGrp + (col & 3) * 64 + half * 16;

  if (ntiles > 0) issue(0, kb);
  if (ntiles > 1) issue(1, kb + kSubBytes);

  // ---- A fragments: the 32 query rows of this block, in registers for the whole sweep
  Frag afrag[KS];
  {
    const int mrow = rb * 32 + col;
    const int a_w = mrow >> gsV, a_g = mrow & (GpV - 1);
    const bool a_ok = seq_ok && a_w < p.W && a_g < p.G;
    const char* qrow = p.q + ((int64_t)l * p.q_sl + (int64_t)seq * p.q_ss +
                              ((int64_t)a_w * p.Hq + (int64_t)h * p.G + a_g) * p.D) * T::bytes;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int k0 = s * M::KPI + half * M::EPL;
      if (a_ok && k0 < p.D) afrag[s] = *(const Frag*)(qrow + (int64_t)k0 * T::bytes);
      else zero_frag<T>(afrag[s]);
    }
  }
  // the sweep counts its own loads with s_waitcnt: the query loads must be out of the way.  They
  // were issued after the first two K blocks, so waiting for them waits for those blocks too.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(afrag[s]));

  ZP_STAMP();
  const int row0 = rb * 32 + half * 4;   // rows of this lane: row0 + (r/4)*8 + r%4
  uint32_t lg[kResTiles * 8];
  float run[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) run[r] = -INFINITY;

  // ---- the sweep: products, causal mask, running maximum, rounded logits into registers.
  // Software-pipelined inside the wave: the products of block it+1 are issued before the
  // vector work on block it, so the matrix core runs under it.
  auto products = [&](int it) {
    const char* cur = kb + (it & 1) * kSubBytes + rd_off;
    f32x16_t acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int s0 = 0; s0 < KS; s0 += 4) {
      Frag bfr[4];
#pragma unroll
      for (int s = 0; s < 4; ++s)
        bfr[s] = *(const Frag*)(cur + ((s0 + s) >> 1) * 256 + ((s0 + s) & 1) * 32);
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = M::mma(afrag[s0 + s], bfr[s], acc);
    }
    return acc;
  };
  f32x16_t acc_cur;
  if (ntiles > 0) acc_cur = products(0);
  // every fragment of block 0 is in registers: block 2 may overwrite it
  asm volatile("" ::: "memory");
  if (ntiles > 2) issue(2, kb);
#pragma unroll
  for (int it = 0; it < kResTiles; ++it) {
    if (it < ntiles) {
      f32x16_t acc_next;
      if (it + 1 < ntiles) {
        // block it+1 has landed once at most the 8 loads of block it+2 are outstanding
        if (it + 1 >= 2) {
          if (it + 2 < ntiles) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(ZP_DMA_N) : "memory");
          else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        acc_next = products(it + 1);
        asm volatile("" ::: "memory");
        if (it + 3 < ntiles) issue(it + 3, kb + ((it + 1) & 1) * kSubBytes);
      }
      f32x16_t acc = acc_cur;
      const int vp = tile_page(it);
      const int vs = page_word(myinfo.y, vp);
      const int toff = (it - vp * tiles_per_page) * 128 + wtok;
      if (((vs >> 30) & 1) && (toff + 31 > p.BS - p.W)) {   // causal mask: tail of the last page
        const int slot = toff + col;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int w = (row0 + (r >> 2) * 8 + (r & 3)) >> gsV;
          if (slot > p.BS - p.W + w) acc[r] = -INFINITY;
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) run[r] = vmax(run[r], acc[r]);
#pragma unroll
      for (int r = 0; r < 16; r += 2)
        lg[it * 8 + (r >> 1)] = P2::pack(acc[r] * p.scale, acc[r + 1] * p.scale);
      if (it + 1 < ntiles) acc_cur = acc_next;
    }
  }

  ZP_STAMP();
  // ---- row maximum over the lanes of a row and the four waves
  auto row_slot = [&](int r) { return (r >> 2) * 8 + half * 4 + (r & 3); };
  float mx[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float v = half_max(run[r]);
    run[r] = v;
    if (col == 0) stat[wave * 32 + row_slot(r)] = v;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float v = run[r];
#pragma unroll
    for (int w2 = 1; w2 < kWaves; ++w2) v = fmaxf(v, stat[((wave + w2) % kWaves) * 32 + row_slot(r)]);
    mx[r] = Elem<T>::rnd(v * p.scale);
  }
  __syncthreads();

  ZP_STAMP();
  // ---- x = rounded(logit - max) back into the registers, row sums of exp(x)
#pragma unroll
  for (int r = 0; r < 16; ++r) run[r] = 0.f;
#pragma unroll
  for (int it = 0; it < kResTiles; ++it) {
    if (it < ntiles) {
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const uint32_t w = lg[it * 8 + q];
        const uint32_t x = P2::pack(P2::lo(w) - mx[2 * q], P2::hi(w) - mx[2 * q + 1]);
        lg[it * 8 + q] = x;
        run[2 * q] += exp_neg(P2::lo(x));
        run[2 * q + 1] += exp_neg(P2::hi(x));
      }
    }
  }
  ZP_STAMP();
  float cl[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float v = half_sum(run[r]);
    run[r] = v;
    if (col == 0) stat[wave * 32 + row_slot(r)] = v;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    // the four waves' sums are added in wave order, whichever wave does it
    float v = stat[row_slot(r)];
#pragma unroll
    for (int w2 = 1; w2 < kWaves; ++w2) v += stat[w2 * 32 + row_slot(r)];
    const int m = row0 + (r >> 2) * 8 + (r & 3);
    const bool ok = (m >> gsV) < p.W && (m & (GpV - 1)) < p.G;
    cl[r] = ok ? -__builtin_amdgcn_logf(v) : -INFINITY;   // rows outside the window or group never win a maximum
  }

  ZP_STAMP();
  // ---- output: p = 2^(x log2(e) - log2(sum)), group maximum, this block's share of the window sum
  float* part = p.part + ((int64_t)item * p.RB + rb) * Tn + wtok + col;
#pragma unroll
  for (int it = 0; it < kResTiles; ++it) {
    if (it < ntiles) {
      float pv[16];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const uint32_t x = lg[it * 8 + q];
        pv[2 * q] = __builtin_fmaf(P2::lo(x), 1.44269504088896340736f, cl[2 * q]);
        pv[2 * q + 1] = __builtin_fmaf(P2::hi(x), 1.44269504088896340736f, cl[2 * q + 1]);
      }
      const float red = group_window_reduce<T>(pv, GpV, rmaxV);
      const int vp = tile_page(it);
      const int j = page_word(myinfo.y, vp) & 0xffff;
      const int toff = (it - vp * tiles_per_page) * 128;
      if (half == 0) __builtin_nontemporal_store(red, part + j * p.BS + toff);
    }
  }
  ZP_STAMP();
#ifdef ZP_RES_STAMP
  if (tid == 0) {
    long long* dst = (long long*)(p.part + (int64_t)p.n_items * p.RB * Tn) + (int64_t)(item * p.RB + rb) * 8;
    for (int i = 0; i < 7; ++i) dst[i] = stamp[i];
    dst[7] = wall_clock64() - wall0;
  }
#endif
#undef ZP_STAMP
}

// ------------------------------------------------------------------ fp32 caches: one sweep
// The same structure for fp32 caches.  An fp32 logit fills a register, so a unit is 16 query rows
// (v_mfma_f32_16x16x4_f32: lane (c, q) = (lane % 16, lane / 16) holds row / token c of the
// operands at contraction index q and rows 4 q .. 4 q + 3 of token c of the result); wave t owns
// tokens [64 i + 16 t, +16) of every 64-token tile i, four logits per tile and lane, 160 registers
// for 40 tiles.  fp32 has no rounding chain: exp(logit - max) replaces the logit in its register
// while the row sums accumulate, and the output pass is one multiplication per entry.
//   * The contraction index is free as long as both operands agree: step 4 j + i of lane group q
//     takes element 16 j + 4 q + i, so a lane's operands for four steps are 16 consecutive bytes.
//   * A load instruction fills 1 KB of LDS with two key rows (32 pieces of 16 bytes each): piece g
//     of row r of a pair at ((g / 16) * 32 + (g % 16) * 2 + r) * 16, pairs 1056 bytes apart, so the
//     sixteen lanes that read one piece of sixteen consecutive rows fall into sixteen different
//     16-byte bank groups.
constexpr int kF32Tiles = 40;              // 64-token tiles of a row: at most 2 560 tokens
constexpr int kF32Pair = 1056;             // bytes from one pair of staged key rows to the next
constexpr int kF32Sub = 8 * kF32Pair;      // a wave's block of 16 key rows
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <int GPC, int RMAXC, int TPP>
__global__ __launch_bounds__(kThreads, 2) void score_resident_f32_kernel(ScoreArgs p) {
  const int GpV = GPC > 0 ? GPC : p.Gp;
  const int gsV = GPC == 8 ? 3 : GPC == 4 ? 2 : GPC == 2 ? 1 : p.gs;
  const bool rmaxV = RMAXC >= 0 ? (RMAXC != 0) : (p.reduce_max != 0);

  extern __shared__ __align__(16) char smem[];
  float* stat = (float*)(smem + kWaves * 2 * kF32Sub);   // [kWaves][16] row maxima, then row sums

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kq = lane >> 4, col = lane & 15;
  // unit -> (item, row block), as in the 16-bit kernel: the row blocks of an item side by side on
  // one XCD
  const int xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
  const int rb = loc % p.RB;
  const int item = (loc / p.RB) * 8 + xcd;
  if (item >= p.n_items) return;
  const int h = item % p.Hkv;
  const int b = (item / p.Hkv) % p.B;
  const int l = item / (p.Hkv * p.B);
  const int Tn = p.NB * p.BS;

  // per-wave list of usable pages: entry n in lane n as (page id, table index | last << 30)
  const int code = lane < p.NB ? p.table[(int64_t)b * p.NB + lane] : -1;
  int seq = p.seq_idx[b];
  int2 myinfo;
  int nvalid;
  {
    const int pid = page_is_pad(code) ? -1 : page_id(code);
    const bool ok = pid >= 0 && pid < p.num_pages;
    const unsigned long long okm = __builtin_amdgcn_ballot_w64(ok);
    nvalid = __builtin_popcountll(okm);
    const int dst = ok ? __builtin_popcountll(okm & lanemask_lt())
                       : nvalid + __builtin_popcountll(~okm & lanemask_lt());
    myinfo.x = __builtin_amdgcn_ds_permute(dst << 2, pid);
    myinfo.y = __builtin_amdgcn_ds_permute(dst << 2, lane | (page_is_last(code) ? (1 << 30) : 0));
  }
  const int dpieces = p.D / 4;               // 16-byte pieces of a key row
  char* kb = smem + wave * 2 * kF32Sub;      // this wave's two key blocks
  if (dpieces < 32) {   // the tail of every staged row must read as zero
    for (int i = lane; i < 2 * kF32Sub / 4; i += 64) ((uint32_t*)kb)[i] = 0u;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  const bool seq_ok = seq >= 0 && seq < p.max_seqs;
  if (!seq_ok) seq = 0;

  const int tiles_per_page = TPP > 0 ? TPP : p.BS / 64;
  const int ntiles = nvalid * tiles_per_page;
  auto tile_page = [&](int tile) { return tile / (TPP > 0 ? TPP : tiles_per_page); };
  auto page_word = [&](int v, int vp) {   // entry vp of the list, wave-uniform
    if constexpr (TPP > 0) return __builtin_amdgcn_readlane(v, vp);
    else return __builtin_amdgcn_readfirstlane(__builtin_amdgcn_ds_bpermute(vp << 2, v));
  };
  const int64_t k_row = (int64_t)p.Hkv * p.D * 4;
  const char* kbase = p.k + (l * p.k_sl) * 4 + (int64_t)h * p.D * 4;
  const int wtok = wave * 16;   // this wave's tokens inside a tile

  // ---- staging: a load instruction moves two rows; lane -> (row of the pair, piece)
  const int st_g = (lane >> 5) * 16 + ((lane & 31) >> 1), st_r = lane & 1;
  const int st_off = (int)(st_r * k_row + st_g * 16);
  const bool st_ok = st_g < dpieces;
  const int pair_step = (int)(2 * k_row);
  typedef void __attribute__((address_space(3))) * lptr_t;
  auto issue = [&](int tile, char* buf) {
    const int vp = tile_page(tile);
    const int pid = page_word(myinfo.x, vp);
    const int toff = (tile - vp * tiles_per_page) * 64 + wtok;
    const char* src = kbase + (int64_t)pid * p.k_sp * 4 + (int64_t)toff * k_row;
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, (int)(16 * k_row), 0x00020000);
    if (st_ok) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(buf + i * kF32Pair), 16, st_off,
                                                 i * pair_step, 0, 0);
    }
  };
  // operands of steps 4 j .. 4 j + 3 of this lane's token: base + (j / 4) * 512 + (j % 4) * 128
  const int rd_off = (col >> 1) * kF32Pair + kq * 32 + (col & 1) * 16;

  if (ntiles > 0) issue(0, kb);
  if (ntiles > 1) issue(1, kb + kF32Sub);

  // ---- A operands: query row `col` of this block at this lane group's contraction indices
  f32x4_t aq[8];
  {
    const int mrow = rb * 16 + col;
    const int a_w = mrow >> gsV, a_g = mrow & (GpV - 1);
    const bool a_ok = seq_ok && a_w < p.W && a_g < p.G;
    const char* qrow = p.q + ((int64_t)l * p.q_sl + (int64_t)seq * p.q_ss +
                              ((int64_t)a_w * p.Hq + (int64_t)h * p.G + a_g) * p.D) * 4;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k0 = 16 * j + 4 * kq;
      if (a_ok && k0 < p.D) aq[j] = *(const f32x4_t*)(qrow + (int64_t)k0 * 4);
      else aq[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  }
  // the sweep counts its own loads with s_waitcnt: the query loads must be out of the way.  They
  // were issued after the first two key blocks, so waiting for them waits for those blocks too.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int j = 0; j < 8; ++j) asm volatile("" : "+v"(aq[j]));

  const int row0 = rb * 16 + kq * 4;   // rows of this lane: row0 + r
  float lg[kF32Tiles * 4];
  float run[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) run[r] = -INFINITY;

  // ---- the sweep: products, causal mask, running maximum, logits into registers; the products
  // of block it+1 are issued before the vector work on block it
  auto products = [&](int it) {
    const char* cur = kb + (it & 1) * kF32Sub + rd_off;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j0 = 0; j0 < 8; j0 += 4) {
      f32x4_t bf[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[j] = *(const f32x4_t*)(cur + ((j0 + j) >> 2) * 512 + ((j0 + j) & 3) * 128);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(aq[j0 + j][i], bf[j][i], acc, 0, 0, 0);
      }
    }
    return acc;
  };
  f32x4_t acc_cur = {0.f, 0.f, 0.f, 0.f};
  if (ntiles > 0) acc_cur = products(0);
  // every operand of block 0 is in registers: block 2 may overwrite it
  asm volatile("" ::: "memory");
  if (ntiles > 2) issue(2, kb);
#pragma unroll
  for (int it = 0; it < kF32Tiles; ++it) {
    if (it < ntiles) {
      f32x4_t acc_next = {0.f, 0.f, 0.f, 0.f};
      if (it + 1 < ntiles) {
        // block it+1 has landed once at most the 8 loads of block it+2 are outstanding
        if (it + 1 >= 2) {
          if (it + 2 < ntiles) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
          else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        acc_next = products(it + 1);
        asm volatile("" ::: "memory");
        if (it + 3 < ntiles) issue(it + 3, kb + ((it + 1) & 1) * kF32Sub);
      }
      f32x4_t acc = acc_cur;
      const int vp = tile_page(it);
      const int vs = page_word(myinfo.y, vp);
      const int toff = (it - vp * tiles_per_page) * 64 + wtok;
      if (((vs >> 30) & 1) && (toff + 15 > p.BS - p.W)) {   // causal mask: tail of the last page
        const int slot = toff + col;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int w = (row0 + r) >> gsV;
          if (slot > p.BS - p.W + w) acc[r] = -INFINITY;
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        run[r] = vmax(run[r], acc[r]);
        lg[it * 4 + r] = acc[r] * p.scale;
      }
      if (it + 1 < ntiles) acc_cur = acc_next;
    }
  }

  // ---- row maximum over the 16 tokens of a lane group and the four waves
  float mx[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float v = row16_max(run[r]);
    run[r] = v;
    if (col == 0) stat[wave * 16 + kq * 4 + r] = v;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float v = run[r];
#pragma unroll
    for (int w2 = 1; w2 < kWaves; ++w2) v = fmaxf(v, stat[((wave + w2) % kWaves) * 16 + kq * 4 + r]);
    mx[r] = v * p.scale;
  }
  __syncthreads();

  // ---- exp(logit - max) back into the registers, row sums
#pragma unroll
  for (int r = 0; r < 4; ++r) run[r] = 0.f;
#pragma unroll
  for (int it = 0; it < kF32Tiles; ++it) {
    if (it < ntiles) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = exp_neg(lg[it * 4 + r] - mx[r]);
        lg[it * 4 + r] = e;
        run[r] += e;
      }
    }
  }
  float inv[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float v = row16_sum(run[r]);
    if (col == 0) stat[wave * 16 + kq * 4 + r] = v;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    // the four waves' sums are added in wave order, whichever wave does it
    float v = stat[kq * 4 + r];
#pragma unroll
    for (int w2 = 1; w2 < kWaves; ++w2) v += stat[w2 * 16 + kq * 4 + r];
    const int m = row0 + r;
    const bool ok = (m >> gsV) < p.W && (m & (GpV - 1)) < p.G;
    inv[r] = ok ? 1.f / v : 0.f;   // rows outside the window or group contribute 0 (probabilities are >= 0)
  }

  // ---- output: p = e / sum, group maximum, this block's share of the window sum (or maximum)
  float* part = p.part + ((int64_t)item * p.RB + rb) * Tn + wtok + col;
#pragma unroll
  for (int it = 0; it < kF32Tiles; ++it) {
    if (it < ntiles) {
      float pv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) pv[r] = lg[it * 4 + r] * inv[r];
      // a lane's four rows are consecutive: groups of 1, 2 or 4 rows are whole inside the lane,
      // groups of 8 / 16 rows span two / four lane groups
      float red;
      if (GpV == 1) {
        red = rmaxV ? vmax4(pv[0], pv[1], pv[2], pv[3]) : (pv[0] + pv[1]) + (pv[2] + pv[3]);
      } else if (GpV == 2) {
        const float g0 = vmax(pv[0], pv[1]), g1 = vmax(pv[2], pv[3]);
        red = rmaxV ? vmax(g0, g1) : g0 + g1;
      } else {
        red = vmax4(pv[0], pv[1], pv[2], pv[3]);
      }
      {
        const float o = lane_xor16(red);
        red = (GpV >= 8 || rmaxV) ? vmax(red, o) : red + o;
      }
      {
        const float o = lane_xor32(red);
        red = (GpV >= 16 || rmaxV) ? vmax(red, o) : red + o;
      }
      const int vp = tile_page(it);
      const int j = page_word(myinfo.y, vp) & 0xffff;
      const int toff = (it - vp * tiles_per_page) * 64;
      if (kq == 0) __builtin_nontemporal_store(red, part + j * p.BS + toff);
    }
  }
}

// Adds the row blocks' window partials of every (layer, sequence, head) in block order, divides by
// the window length, rounds to the cache dtype; pad pages score exactly 0.
template <typename T>
__global__ __launch_bounds__(256) void score_combine_kernel(const float* __restrict__ part,
                                                            void* __restrict__ out,
                                                            const int32_t* __restrict__ table,
                                                            int B, int NB, int BS, int Hkv, int RB,
                                                            int W, int num_pages, int rmax) {
  // four consecutive tokens per thread (a page is a multiple of 128 tokens)
  const int item = blockIdx.x;
  const int b = (item / Hkv) % B;
  const int Tn = NB * BS;
  const int t = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (t >= Tn) return;
  const int code = table[(int64_t)b * NB + t / BS];
  const int pid = page_is_pad(code) ? -1 : page_id(code);
  typedef float f4 __attribute__((ext_vector_type(4)));
  f4 v = {0.f, 0.f, 0.f, 0.f};
  if (pid >= 0 && pid < num_pages) {
    const float* src = part + (int64_t)item * RB * Tn + t;
    v = __builtin_nontemporal_load((const f4*)src);
    for (int r = 1; r < RB; ++r) {
      const f4 o = __builtin_nontemporal_load((const f4*)(src + (int64_t)r * Tn));
      if (rmax) { v.x = fmaxf(v.x, o.x); v.y = fmaxf(v.y, o.y); v.z = fmaxf(v.z, o.z); v.w = fmaxf(v.w, o.w); }
      else { v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w; }
    }
    if (!rmax) {
      v.x = Elem<T>::rnd(v.x / (float)W); v.y = Elem<T>::rnd(v.y / (float)W);
      v.z = Elem<T>::rnd(v.z / (float)W); v.w = Elem<T>::rnd(v.w / (float)W);
    }
  }
  const int64_t o = (int64_t)item * Tn + t;
  if constexpr (T::bytes == 2) {
    uint16_t* dst = (uint16_t*)out + o;
    if constexpr (std::is_same<T, BF16>::value) {
      const uint2 w = make_uint2(float_to_bf16_bits(v.x) | ((uint32_t)float_to_bf16_bits(v.y) << 16),
                                 float_to_bf16_bits(v.z) | ((uint32_t)float_to_bf16_bits(v.w) << 16));
      *(uint2*)dst = w;
    } else {
      const uint2 w = make_uint2(float_to_f16_bits(v.x) | ((uint32_t)float_to_f16_bits(v.y) << 16),
                                 float_to_f16_bits(v.z) | ((uint32_t)float_to_f16_bits(v.w) << 16));
      *(uint2*)dst = w;
    }
  } else {
    *(f4*)((float*)out + o) = v;
  }
}

}  // namespace

static int pow2_ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

// Can the register-resident kernel take this shape (16-bit caches only; the caller checks the
// dtype, the logits request and the sign of the scale)?
static bool resident_shape_ok(int NB, int BS, int Hkv, int Hq, int D) {
  if (Hkv <= 0 || Hq <= 0 || Hq % Hkv != 0) return false;
  const int Gp = pow2_ceil(Hq / Hkv);
  return BS % 128 == 0 && (int64_t)NB * (BS / 128) <= kResTiles && NB <= 64 && Gp <= 32 &&
         D <= kDmax && (D * 2) % 16 == 0;
}

// Scratch the three-sweep kernel cannot do without (window x group beyond 128 rows).
static int64_t sweep_workspace(int L, int B, int NB, int BS, int Hkv, int Hq, int W) {
  const int Gp = pow2_ceil(Hq / Hkv);
  const int RB = (W * Gp + 31) / 32;
  if (RB <= kRowWaves) return 0;
  return (int64_t)L * B * Hkv * NB * BS * 4;
}

// fp32 caches: pages in whole 64-token tiles, at most 40 tiles, groups of at most 16 rows.
static bool resident_f32_shape_ok(int NB, int BS, int Hkv, int Hq, int D) {
  if (Hkv <= 0 || Hq <= 0 || Hq % Hkv != 0) return false;
  const int Gp = pow2_ceil(Hq / Hkv);
  return BS % 64 == 0 && (int64_t)NB * (BS / 64) <= kF32Tiles && NB <= 64 && Gp <= 16 &&
         D <= kDmax && D % 4 == 0;
}

// Bytes of fp32 window partials the one-sweep kernel of a dtype needs (0: the shape takes three
// sweeps): one partial per token and block of 32 (16-bit caches) or 16 (fp32) query rows.
static int64_t resident_need(int L, int B, int NB, int BS, int Hkv, int Hq, int W, int dtype) {
  if (Hkv <= 0 || Hq <= 0 || Hq % Hkv != 0) return 0;
  const int Gp = pow2_ceil(Hq / Hkv);
  if (dtype == ZP_F32) {
    if (!resident_f32_shape_ok(NB, BS, Hkv, Hq, kDmax)) return 0;
    return (int64_t)L * B * Hkv * ((W * Gp + 15) / 16) * NB * BS * 4;
  }
  if (!resident_shape_ok(NB, BS, Hkv, Hq, kDmax)) return 0;
  return (int64_t)L * B * Hkv * ((W * Gp + 31) / 32) * NB * BS * 4;
}

extern "C" int64_t zp_attention_score_workspace_for(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                                    int32_t Hkv, int32_t Hq, int32_t W, int32_t dtype) {
  if (Hkv <= 0 || Hq <= 0 || L < 0 || B < 0 || NB <= 0 || BS <= 0 || W <= 0) return 0;
  if (dtype < ZP_BF16 || dtype > ZP_F32) return -1;
  const int64_t floor_bytes = sweep_workspace(L, B, NB, BS, Hkv, Hq, W);
  const int64_t res = resident_need(L, B, NB, BS, Hkv, Hq, W, dtype);
  return res > floor_bytes ? res : floor_bytes;
}

extern "C" int64_t zp_attention_score_workspace(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                                int32_t Hkv, int32_t Hq, int32_t W) {
  const int64_t a = zp_attention_score_workspace_for(L, B, NB, BS, Hkv, Hq, W, ZP_BF16);
  const int64_t b = zp_attention_score_workspace_for(L, B, NB, BS, Hkv, Hq, W, ZP_F32);
  return a > b ? a : b;
}

int64_t zp_attention_score_workspace_floor(int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                                           int32_t Hq, int32_t W) {
  if (Hkv <= 0 || Hq <= 0) return 0;
  return sweep_workspace(L, B, NB, BS, Hkv, Hq, W);
}

extern "C" int zp_attention_score(const void* k_cache, const void* query_cache,
                                  const int32_t* seq_idx, const int32_t* block_table,
                                  void* scores_out, void* logits_out, int32_t L, int32_t B,
                                  int32_t NB, int32_t BS, int32_t Hkv, int32_t Hq, int32_t D,
                                  int32_t W, int32_t num_pages, int32_t max_seqs, int64_t k_sl,
                                  int64_t k_sp, int64_t q_sl, int64_t q_ss, float softmax_scale,
                                  int32_t reduced, int32_t dtype, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  ZP_REQUIRE(k_cache && query_cache && seq_idx && block_table && scores_out,
             "attention_score: null pointer");
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0 && Hq > 0 && D > 0 && W > 0,
             "attention_score: bad dims");
  ZP_REQUIRE(Hq % Hkv == 0, "attention_score: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "attention_score: unknown dtype tag %d", dtype);
  ZP_REQUIRE(reduced == ZP_REDUCE_MEAN || reduced == ZP_REDUCE_MAX,
             "attention_score: unknown reduction %d", reduced);
  ZP_REQUIRE(W <= BS, "attention_score: window %d longer than a page of %d", W, BS);
  const int es = zp_dtype_bytes(dtype);
  const int TN = dtype == ZP_F32 ? Mma<F32>::TN : Mma<BF16>::TN;
  if (!(D <= kDmax && (D * es) % 16 == 0)) {
    zp_set_error("attention_score: head_dim %d unsupported (need <= %d and a multiple of %d)", D,
                 kDmax, 16 / es);
    return ZP_EUNSUPPORTED;
  }
  if (BS % TN != 0) {
    zp_set_error("attention_score: page size %d is not a multiple of %d", BS, TN);
    return ZP_EUNSUPPORTED;
  }
  const int G = Hq / Hkv, Gp = pow2_ceil(G);
  if (Gp > 32) {
    zp_set_error("attention_score: GQA group %d unsupported (max 32)", G);
    return ZP_EUNSUPPORTED;
  }
  ZP_REQUIRE(((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)query_cache % 16) == 0 &&
                 (k_sl * es) % 16 == 0 && (k_sp * es) % 16 == 0 && (q_sl * es) % 16 == 0 &&
                 (q_ss * es) % 16 == 0,
             "attention_score: caches must be 16-byte aligned");
  ZP_REQUIRE(NB <= 0xffff, "attention_score: too many pages per sequence");
  if (L == 0 || B == 0) return ZP_OK;
  const int RB = (W * Gp + 31) / 32;
  const int64_t need = sweep_workspace(L, B, NB, BS, Hkv, Hq, W);
  // One sweep over K with the logits in registers when the shape allows it and the caller
  // brought the scratch for the window partials; three sweeps otherwise.
  const int64_t res_need = resident_need(L, B, NB, BS, Hkv, Hq, W, dtype);
  const bool res_common = !logits_out && softmax_scale > 0.f && workspace && res_need > 0 &&
                          workspace_bytes >= res_need && ((uintptr_t)workspace % 16) == 0 &&
                          (int64_t)L * B * Hkv < ((int64_t)1 << 27);
  const bool resident = es == 2 && res_common && resident_shape_ok(NB, BS, Hkv, Hq, D);
  const bool resident32 = es == 4 && res_common && resident_f32_shape_ok(NB, BS, Hkv, Hq, D);
  ZP_REQUIRE(resident || resident32 || need == 0 || (workspace && workspace_bytes >= need),
             "attention_score: workspace of %lld bytes required", (long long)need);

  ScoreArgs a;
  a.k = (const char*)k_cache; a.q = (const char*)query_cache; a.seq_idx = seq_idx;
  a.table = block_table; a.out = scores_out; a.logits = logits_out; a.ws = (float*)workspace;
  a.L = L; a.B = B; a.NB = NB; a.BS = BS; a.Hkv = Hkv; a.Hq = Hq; a.G = G; a.Gp = Gp; a.D = D;
  a.W = W; a.num_pages = num_pages; a.max_seqs = max_seqs;
  a.k_sl = k_sl; a.k_sp = k_sp; a.q_sl = q_sl; a.q_ss = q_ss;
  a.scale = softmax_scale; a.reduce_max = reduced == ZP_REDUCE_MAX; a.RB = RB;
  a.gs = 0;
  while ((1 << a.gs) < Gp) ++a.gs;
  a.RW = RB >= 3 ? kRowWaves : RB;
  if (a.RW < kWaves / (TN / 32)) a.RW = kWaves / (TN / 32);  // every wave needs >= 1 subtile

  hipStream_t st = (hipStream_t)stream;
  a.n_items = L * B * Hkv;
  a.part = (float*)workspace;
  if (resident) {
    const size_t smem = (size_t)kWaves * 2 * kSubBytes + sizeof(float) * kWaves * 32;
    const unsigned units = (unsigned)(((int64_t)a.n_items + 7) / 8 * 8 * RB);
    const dim3 cgrid((unsigned)a.n_items, (unsigned)((NB * BS / 4 + 255) / 256));
#define ZP_RESIDENT_LAUNCH(TT)                                                                   \
  do {                                                                                           \
    void (*fn)(ScoreArgs) = score_resident_kernel<TT, 0, -1, 0>;                                 \
    if (Gp == 4 && !a.reduce_max && BS == 256) fn = score_resident_kernel<TT, 4, 0, 2>;          \
    if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize,         \
                            (int)smem) != hipSuccess) {                                          \
      zp_set_error("attention_score: cannot reserve %zu bytes of LDS", smem);                    \
      return ZP_EHIP;                                                                            \
    }                                                                                            \
    hipLaunchKernelGGL(fn, dim3(units), dim3(kThreads), smem, st, a);                            \
    hipLaunchKernelGGL(score_combine_kernel<TT>, cgrid, dim3(256), 0, st, a.part, scores_out,    \
                       block_table, B, NB, BS, Hkv, RB, W, num_pages, a.reduce_max);             \
  } while (0)
    if (dtype == ZP_BF16) ZP_RESIDENT_LAUNCH(BF16);
    else ZP_RESIDENT_LAUNCH(F16);
#undef ZP_RESIDENT_LAUNCH
    ZP_LAUNCH_CHECK();
    return ZP_OK;
  }
  if (resident32) {
    a.RB = (W * Gp + 15) / 16;
    const size_t smem = (size_t)kWaves * 2 * kF32Sub + sizeof(float) * kWaves * 16;
    const unsigned units = (unsigned)(((int64_t)a.n_items + 7) / 8 * 8 * a.RB);
    const dim3 cgrid((unsigned)a.n_items, (unsigned)((NB * BS / 4 + 255) / 256));
    void (*fn)(ScoreArgs) = score_resident_f32_kernel<0, -1, 0>;
    if (Gp == 2 && !a.reduce_max && BS == 256) fn = score_resident_f32_kernel<2, 0, 4>;
    else if (Gp == 4 && !a.reduce_max && BS == 256) fn = score_resident_f32_kernel<4, 0, 4>;
    if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) !=
        hipSuccess) {
      zp_set_error("attention_score: cannot reserve %zu bytes of LDS", smem);
      return ZP_EHIP;
    }
    hipLaunchKernelGGL(fn, dim3(units), dim3(kThreads), smem, st, a);
    hipLaunchKernelGGL(score_combine_kernel<F32>, cgrid, dim3(256), 0, st, a.part, scores_out, block_table,
                       B, NB, BS, Hkv, a.RB, W, num_pages, a.reduce_max);
    ZP_LAUNCH_CHECK();
    return ZP_OK;
  }
  dim3 grid((unsigned)((int64_t)L * B * Hkv));
#define ZP_SCORE_LAUNCH()                                                                        \
  do {                                                                                           \
    const size_t smem = 2 * (size_t)Mma<T>::TN * Mma<T>::ROWB +                                  \
                        sizeof(float) * (2 * kRowWaves * Mma<T>::TN + kWaves * 32) + sizeof(int2) * NB; \
    void (*fn)(ScoreArgs) = score_kernel<T, false, 0, -1>;                                       \
    if (logits_out) fn = score_kernel<T, true, 0, -1>;                                           \
    else if (T::bytes == 2 && Gp == 4 && !a.reduce_max) fn = score_kernel<T, false, 4, 0>;       \
    else if (T::bytes == 2 && Gp == 2 && !a.reduce_max) fn = score_kernel<T, false, 2, 0>;       \
    else if (T::bytes == 2 && Gp == 8 && !a.reduce_max) fn = score_kernel<T, false, 8, 0>;       \
    if (smem > 64 * 1024 &&                                                                      \
        hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize,         \
                            (int)smem) != hipSuccess) {                                          \
      zp_set_error("attention_score: cannot reserve %zu bytes of LDS", smem);                    \
      return ZP_EHIP;                                                                            \
    }                                                                                            \
    hipLaunchKernelGGL(fn, grid, dim3(kThreads), smem, st, a);                                   \
  } while (0)
  ZP_DISPATCH_DTYPE(dtype, ZP_SCORE_LAUNCH());
#undef ZP_SCORE_LAUNCH
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}
