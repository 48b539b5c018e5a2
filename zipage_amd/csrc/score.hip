// Ragged attention scorer: softmax(window queries x paged keys), max over the GQA group,
// mean (or max) over the window -- one workgroup per (layer, sequence, kv head), MFMA
// for the QK^T contraction, K tiles staged through double-buffered LDS.
//
// The (Hq, W, T) logits the reference materialises are never written (unless the caller
// asks for them).  The softmax normaliser spans the whole sequence, so the workgroup makes
// three passes over the sequence's pages, recomputing QK^T each time:
//   pass 1  row maximum of the (rounded) logits,
//   pass 2  row sum of exp(rounded(logit - max)),
//   pass 3  p = exp(.) / sum, max over the group, sum over the window, store (the group
//           maximum is taken on the exponents x*log2(e) - log2(sum), one exponential per group).
// Passes 2 and 3 re-read K from L2 / Infinity Cache.  Rounding points follow the
// reference (logits, logit-max, softmax output and the window mean are each rounded to the
// cache dtype), so bf16/fp16 results agree with it to the last bit except where fp32
// accumulation order moves a value across a rounding boundary.
//
// MFMA tiling (wave64, 32x32 tiles): the A operand is a block of 32 query rows, row
// m = w*Gp + g (Gp = GQA group padded to a power of two), held in registers for the
// whole pass; the B operand is 32 tokens of the K tile read from LDS.  In the 32x32
// accumulator layout a lane owns one token column and 16 rows
// ((r/4)*8 + (lane/32)*4 + r%4), so with this row order the group maximum is taken inside
// a lane (plus one cross-half exchange when Gp >= 8) and the window sum is a lane-local
// sum plus one cross-half and one cross-wave (LDS) step.  Wave v of the workgroup owns
// row block v; tiles of 128 (16-bit) or 64 (fp32) tokens are shared by all waves.
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
                for (int r = 0; r < 16; ++r) run[r] = vmax(vmax(run[r], accA[r]), accB[r]);
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
                    q4[q] = vmax(vmax(pv[4 * q], pv[4 * q + 1]), vmax(pv[4 * q + 2], pv[4 * q + 3]));
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
                    red = rmaxV ? vmax(vmax(q4[0], q4[1]), vmax(q4[2], q4[3]))
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
                    red = vmax(vmax(vmax(t8[0], t8[1]), vmax(t8[2], t8[3])),
                                vmax(vmax(t8[4], t8[5]), vmax(t8[6], t8[7])));
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

}  // namespace

static int pow2_ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

extern "C" int64_t zp_attention_score_workspace(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                                int32_t Hkv, int32_t Hq, int32_t W) {
  if (Hkv <= 0 || Hq <= 0) return 0;
  const int Gp = pow2_ceil(Hq / Hkv);
  const int RB = (W * Gp + 31) / 32;
  if (RB <= kRowWaves) return 0;
  return (int64_t)L * B * Hkv * NB * BS * 4;
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
  const int64_t need = zp_attention_score_workspace(L, B, NB, BS, Hkv, Hq, W);
  ZP_REQUIRE(need == 0 || (workspace && workspace_bytes >= need),
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
