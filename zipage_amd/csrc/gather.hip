// Gather / scatter kernels: in-place compaction of surviving K/V (and of the carried
// score cache) into a sequence's fixed page budget, and the query-window ring store.
//
// Compaction (one workgroup per (layer, sequence, kv head)):
//   phase 1  scan the row's keep flags once and build, in LDS, the ordered list of
//            surviving logical token indices (block-wide exclusive scan);
//   phase 2  walk that list in rounds; every thread gathers R 16-byte pieces of K and of
//            V into registers, the workgroup waits for all of its loads and meets at a
//            barrier, then scatters the pieces to their destinations.
// Why this is safe in place: the n-th survivor has logical source index s(n) >= n and
// the list is ascending.  A destination n aliases (by the engine's page-table rule) a
// source position <= n, which is either in the current round (already loaded: the
// barrier orders load-before-store) or in an earlier round.  Later rounds only read
// positions > every position written so far, so rounds need no ordering between them
// and the next round's loads overlap the current round's stores.
// The one-call pipeline moves the carried scores of the survivors in the same launch (same list,
// rounds of their own after the K/V rounds); zp_compress_score is the launch of its own.
#include "common.h"
#include <type_traits>

namespace {

constexpr int kThreads = 256;
constexpr int kCompactR = 8;   // 16-byte pieces each thread gathers per round
#ifndef ZP_SPLIT_ROWS
#define ZP_SPLIT_ROWS 1024
#endif
constexpr int kSplitKvRows = ZP_SPLIT_ROWS;   // up to this many (layer, sequence, head) rows K and V get workgroups of their own
// native vector types keep the staged pieces in VGPRs
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int block_exclusive_scan(int v, int* total, int* lds) {
  const int lane = lane_id(), w = wave_id();
  int inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int t = __shfl_up(inc, o, 64);
    if (lane >= o) inc += t;
  }
  if (lane == 63) lds[w] = inc;
  __syncthreads();
  int woff = 0, tot = 0;
#pragma unroll
  for (int i = 0; i < kThreads / 64; ++i) {
    int c = lds[i];
    if (i < w) woff += c;
    tot += c;
  }
  *total = tot;
  return woff + inc - v;
}

struct CompactArgs {
  char* a;             // key (or score cache)
  char* b;             // value (unused when !HAS_B)
  const uint8_t* flag;
  const int32_t* table;
  const int32_t* target;
  int B, NB, BS, Hkv, num_pages, target_width;
  int n_items;         // L*B*Hkv
  int lpv;             // pieces per token vector
  int lpv_shift;       // log2(lpv) or -1
  int bs_shift;        // log2(BS) or -1
  int64_t a_sl, a_sp, a_ss, a_sh;  // byte strides: layer, page, slot, head
  int64_t b_sl, b_sp, b_ss, b_sh;
  // score compaction only: when set, the value of logical token s of row (l, b, h) is read from
  // rows[((l*B + b)*Hkv + h)*T + s] (elements of sizeof(P)) instead of from `a` through the table
  const char* rows;
  // K/V compaction with the carried scores in the same launch (CES != 0): the score cache, its
  // byte strides, and optionally the rows to read the scores from (as `rows` above)
  char* c;
  const char* c_rows;
  int64_t c_sl, c_sp, c_ss, c_sh;
  // !HAS_B with split_kv: the grid is twice n_items; workgroups n_items .. 2 n_items - 1 move
  // `b` (the values) with the same list, the first n_items move `a` (and the carried scores)
  int split_kv;
};

// Survivors are written once and not read again by this kernel: non-temporal stores keep them
// from displacing the gather's source lines in L2 (measured at 256 sequences on one allocation:
// 704 -> 686 us per launch; non-temporal loads on top: 720 us).
#define ZP_NT_LOAD(ptr) (*(ptr))
#define ZP_NT_STORE(v, ptr) __builtin_nontemporal_store(v, ptr)
// POW2: page size and pieces-per-vector are powers of two, so every index split is a shift.
// CES: bytes of a carried-score element moved along with K and V by the same survivor list (0: none).
template <typename P, int R, bool HAS_B, bool POW2, int CES = 0>
__global__ __launch_bounds__(kThreads) void compact_kernel(CompactArgs p) {
  extern __shared__ __align__(16) char smem[];
  __shared__ int scan_lds[kThreads / 64];
  const int T = p.NB * p.BS;
  uint16_t* list = (uint16_t*)smem;
  int* tab = (int*)(smem + (((size_t)T * 2 + 15) & ~(size_t)15));
  int* tgt = tab + p.NB;

  const int tid = threadIdx.x;
  // Workgroup id == item: ids are dealt round-robin to the 8 XCDs, so with 8 kv heads every XCD
  // works on one head's 256-byte slice of the token rows.  Measured against giving each XCD a
  // contiguous range of items (all heads of a sequence on one XCD: 2.5 % slower) and against
  // rotating the head index by the sequence index (4 % slower), inside one allocation.
  const int which = (!HAS_B && p.split_kv && (int)blockIdx.x >= p.n_items) ? 1 : 0;
  const int item = (int)blockIdx.x - which * p.n_items;
  if (item >= p.n_items) return;
  const int h = item % p.Hkv;
  const int b = (item / p.Hkv) % p.B;
  const int l = item / (p.Hkv * p.B);

  for (int i = tid; i < p.NB; i += kThreads) {
    int code = p.table[(int64_t)b * p.NB + i];
    int pid = page_is_pad(code) ? -1 : page_id(code);
    tab[i] = (pid >= 0 && pid < p.num_pages) ? pid : -1;
  }
  for (int i = tid; i < p.target_width; i += kThreads) {
    int t = p.target[(int64_t)b * p.target_width + i];
    tgt[i] = (t >= 0 && t < p.num_pages) ? t : -1;
  }
  __syncthreads();

  // ---- phase 1: ordered survivor list
  const int chunk = (T + kThreads - 1) / kThreads;
  const int s0 = min(tid * chunk, T), s1 = min(s0 + chunk, T);
  const uint8_t* f = p.flag + (((int64_t)l * p.B + b) * p.Hkv + h) * (int64_t)T;
  int cnt = 0;
  auto page_of = [&](int s) { return POW2 ? (s >> p.bs_shift) : (s / p.BS); };
  for (int s = s0; s < s1; ++s) cnt += (f[s] != 0 && tab[page_of(s)] >= 0) ? 1 : 0;
  int total;
  int off = block_exclusive_scan(cnt, &total, scan_lds);
  for (int s = s0; s < s1; ++s)
    if (f[s] != 0 && tab[page_of(s)] >= 0) list[off++] = (uint16_t)s;
  __syncthreads();
  const int cap = p.target_width * p.BS;
  if (total > cap) total = cap;

  // ---- phase 2: gather -> barrier -> scatter, R pieces per thread per round
  const int units = total * p.lpv;
  char* abase = which ? p.b + l * p.b_sl + h * p.b_sh : p.a + l * p.a_sl + h * p.a_sh;
  char* bbase = HAS_B ? p.b + l * p.b_sl + h * p.b_sh : nullptr;
  const int64_t a_sp = which ? p.b_sp : p.a_sp, a_ss = which ? p.b_ss : p.a_ss;
  for (int base = 0; base < units; base += kThreads * R) {
    P ra[R];
    P rb[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      // out-of-range units re-load the last valid piece (never stored): no predicated loads
      const int u = min(base + r * kThreads + tid, units - 1);
      const int i = POW2 ? (u >> p.lpv_shift) : (u / p.lpv), piece = u - i * p.lpv;
      const int s = list[i];
      const int j = page_of(s), slot = s - j * p.BS;
      const int64_t pid = tab[j];
      if (!HAS_B && p.rows)
        ra[r] = *(const P*)(p.rows + ((int64_t)item * T + s) * (int)sizeof(P));
      else
        ra[r] = ZP_NT_LOAD((const P*)(abase + pid * a_sp + slot * a_ss + piece * (int)sizeof(P)));
      if (HAS_B)
        rb[r] = ZP_NT_LOAD((const P*)(bbase + pid * p.b_sp + slot * p.b_ss + piece * (int)sizeof(P)));
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int u = base + r * kThreads + tid;
      if (u < units) {
        const int i = POW2 ? (u >> p.lpv_shift) : (u / p.lpv), piece = u - i * p.lpv;
        const int j = page_of(i), slot = i - j * p.BS;
        const int64_t pid = tgt[j];
        if (pid >= 0) {
          ZP_NT_STORE(ra[r], (P*)(abase + pid * a_sp + slot * a_ss + piece * (int)sizeof(P)));
          if (HAS_B)
            ZP_NT_STORE(rb[r], (P*)(bbase + pid * p.b_sp + slot * p.b_ss + piece * (int)sizeof(P)));
        }
      }
    }
  }
  if (CES != 0 && which == 0) {
    // the carried score of every survivor follows its key: same list, same gather -> barrier ->
    // scatter rounds (the score cache aliases its own targets exactly as the key cache does)
    typedef typename std::conditional<CES == 4, uint32_t, uint16_t>::type E;
    constexpr int RC = 4;
    char* cbase = p.c + l * p.c_sl + h * p.c_sh;
    for (int base = 0; base < total; base += kThreads * RC) {
      E rc[RC];
#pragma unroll
      for (int r = 0; r < RC; ++r) {
        const int s = list[min(base + r * kThreads + tid, total - 1)];
        if (p.c_rows) {
          rc[r] = *(const E*)(p.c_rows + ((int64_t)item * T + s) * CES);
        } else {
          const int j = page_of(s), slot = s - j * p.BS;
          rc[r] = *(const E*)(cbase + (int64_t)tab[j] * p.c_sp + slot * p.c_ss);
        }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
#pragma unroll
      for (int r = 0; r < RC; ++r) {
        const int i = base + r * kThreads + tid;
        if (i < total) {
          const int j = page_of(i), slot = i - j * p.BS;
          const int64_t pid = tgt[j];
          if (pid >= 0) *(E*)(cbase + pid * p.c_sp + slot * p.c_ss) = rc[r];
        }
      }
    }
  }
}

static int log2_exact(int v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

template <typename P, int R, bool HAS_B, bool POW2, int CES = 0>
int launch_compact_impl(CompactArgs a, int L, hipStream_t st) {
  a.n_items = L * a.B * a.Hkv;
  const int T = a.NB * a.BS;
  size_t smem = (((size_t)T * 2 + 15) & ~(size_t)15) + sizeof(int) * (a.NB + a.target_width);
  dim3 grid((unsigned)((int64_t)L * a.B * a.Hkv * (!HAS_B && a.split_kv ? 2 : 1)));
  if (smem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)compact_kernel<P, R, HAS_B, POW2, CES>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      zp_set_error("compaction: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return ZP_EHIP;
    }
  }
  hipLaunchKernelGGL((compact_kernel<P, R, HAS_B, POW2, CES>), grid, dim3(kThreads), smem, st, a);
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}

template <typename P, int R, bool HAS_B, int CES = 0>
int launch_compact(CompactArgs a, int L, hipStream_t st) {
  a.lpv_shift = log2_exact(a.lpv);
  a.bs_shift = log2_exact(a.BS);
  if (a.lpv_shift >= 0 && a.bs_shift >= 0) return launch_compact_impl<P, R, HAS_B, true, CES>(a, L, st);
  return launch_compact_impl<P, R, HAS_B, false, CES>(a, L, st);
}

inline bool aligned_to(int64_t v, int n) { return (v % n) == 0; }

// ------------------------------------------------------------------ query ring store
template <typename P>
__global__ __launch_bounds__(kThreads) void store_query_kernel(
    const char* __restrict__ q, char* __restrict__ qc, const int32_t* __restrict__ sm, int pieces,
    int num_tokens, int max_seqs, int window, int64_t q_st, int64_t c_sseq, int64_t c_sslot,
    int64_t sm_r, int64_t sm_c) {
  const int idx = blockIdx.x;
  const int pos = sm[idx * sm_r];
  const int seq = sm[idx * sm_r + sm_c];
  const int slot = sm[idx * sm_r + 2 * sm_c];
  if (pos < 0 || pos >= num_tokens || seq < 0 || seq >= max_seqs || slot < 0 || slot >= window)
    return;
  const P* src = (const P*)(q + pos * q_st);
  P* dst = (P*)(qc + seq * c_sseq + slot * c_sslot);
  for (int i = threadIdx.x; i < pieces; i += kThreads) dst[i] = src[i];
}

}  // namespace

namespace {
// K/V compaction; with score_cache != nullptr the carried scores move in the same launch when the
// K/V vectors allow 16-byte pieces (otherwise *fused is left false and the caller runs
// zp_compress_score itself).
int compress_kv_impl(void* key, void* value, const uint8_t* flag, const int32_t* block_table,
                     const int32_t* target_block_table, int32_t L, int32_t B, int32_t NB, int32_t BS,
                     int32_t Hkv, int32_t D, int32_t num_pages, int32_t target_width, int64_t k_sl,
                     int64_t k_sp, int64_t k_ss, int64_t k_sh, int64_t v_sl, int64_t v_sp,
                     int64_t v_ss, int64_t v_sh, int32_t dtype, void* score_cache,
                     const void* scores_src, int64_t c_sl, int64_t c_sp, int64_t c_ss, int64_t c_sh,
                     bool* fused, void* stream) {
  ZP_REQUIRE(key && value && flag && block_table && target_block_table, "compress_kv: null pointer");
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0 && D > 0 && target_width > 0,
             "compress_kv: bad dims L=%d B=%d NB=%d BS=%d Hkv=%d D=%d tw=%d", L, B, NB, BS, Hkv, D,
             target_width);
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "compress_kv: unknown dtype tag %d", dtype);
  ZP_REQUIRE((int64_t)NB * BS <= 65536, "compress_kv: NB*BS=%lld exceeds 65536",
             (long long)NB * BS);
  ZP_REQUIRE((int64_t)L * B * Hkv < ((int64_t)1 << 31), "compress_kv: too many (layer, sequence, head) rows");
  if (fused) *fused = false;
  if (L == 0 || B == 0) return ZP_OK;
  const int es = zp_dtype_bytes(dtype);
  CompactArgs a;
  a.a = (char*)key; a.b = (char*)value; a.flag = flag; a.table = block_table;
  a.target = target_block_table; a.rows = nullptr;
  a.B = B; a.NB = NB; a.BS = BS; a.Hkv = Hkv; a.num_pages = num_pages;
  a.target_width = target_width;
  a.a_sl = k_sl * es; a.a_sp = k_sp * es; a.a_ss = k_ss * es; a.a_sh = k_sh * es;
  a.b_sl = v_sl * es; a.b_sp = v_sp * es; a.b_ss = v_ss * es; a.b_sh = v_sh * es;
  a.c = (char*)score_cache; a.c_rows = (const char*)scores_src;
  a.c_sl = c_sl * es; a.c_sp = c_sp * es; a.c_ss = c_ss * es; a.c_sh = c_sh * es;
  const int64_t vec = (int64_t)D * es;
  int piece = 2;
  for (int cand : {16, 8, 4}) {
    bool ok = aligned_to(vec, cand) && aligned_to((int64_t)(uintptr_t)key, cand) &&
              aligned_to((int64_t)(uintptr_t)value, cand);
    for (int64_t s : {a.a_sl, a.a_sp, a.a_ss, a.a_sh, a.b_sl, a.b_sp, a.b_ss, a.b_sh})
      ok = ok && aligned_to(s, cand);
    if (ok) { piece = cand; break; }
  }
  a.lpv = (int)(vec / piece);
  ZP_REQUIRE((int64_t)target_width * BS * a.lpv < (int64_t)1 << 31, "compress_kv: row too large");
  hipStream_t st = (hipStream_t)stream;
  a.split_kv = 0;
  // few rows: keys and values go to workgroups of their own (twice the workgroups per CU to hide
  // the gather's latency: 0.340 against 0.347 ms per step at 64 sequences x 8 heads; with many rows
  // the CUs are full either way and one survivor list per row is cheaper)
  const bool split = piece == 16 && (int64_t)L * B * Hkv <= kSplitKvRows;
  switch (piece) {
    case 16:
      if (score_cache && fused) {
        *fused = true;
        if (split) {
          a.split_kv = 1;
          if (es == 4) return launch_compact<u32x4, 2 * kCompactR, false, 4>(a, L, st);
          return launch_compact<u32x4, 2 * kCompactR, false, 2>(a, L, st);
        }
        if (es == 4) return launch_compact<u32x4, kCompactR, true, 4>(a, L, st);
        return launch_compact<u32x4, kCompactR, true, 2>(a, L, st);
      }
      if (split) {
        a.split_kv = 1;
        return launch_compact<u32x4, 2 * kCompactR, false>(a, L, st);
      }
      return launch_compact<u32x4, kCompactR, true>(a, L, st);
    case 8:  return launch_compact<u32x2, 8, true>(a, L, st);
    case 4:  return launch_compact<uint32_t, 8, true>(a, L, st);
    default: return launch_compact<uint16_t, 8, true>(a, L, st);
  }
}
}  // namespace

extern "C" int zp_compress_kv(void* key, void* value, const uint8_t* flag,
                              const int32_t* block_table, const int32_t* target_block_table,
                              int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                              int32_t D, int32_t num_pages, int32_t target_width,
                              int64_t k_sl, int64_t k_sp, int64_t k_ss, int64_t k_sh,
                              int64_t v_sl, int64_t v_sp, int64_t v_ss, int64_t v_sh,
                              int32_t dtype, void* stream) {
  return compress_kv_impl(key, value, flag, block_table, target_block_table, L, B, NB, BS, Hkv, D,
                          num_pages, target_width, k_sl, k_sp, k_ss, k_sh, v_sl, v_sp, v_ss, v_sh,
                          dtype, nullptr, nullptr, 0, 0, 0, 0, nullptr, stream);
}

// K/V compaction and the compaction of the carried scores (zp_compress_score with the same flags
// and tables) as one launch where the shapes allow it, as the two calls otherwise.
int zp_compress_kv_and_score(void* key, void* value, void* score_cache, const void* scores_src,
                             const uint8_t* flag, const int32_t* block_table,
                             const int32_t* target_block_table, int32_t L, int32_t B, int32_t NB,
                             int32_t BS, int32_t Hkv, int32_t D, int32_t num_pages,
                             int32_t target_width, int64_t k_sl, int64_t k_sp, int64_t k_ss,
                             int64_t k_sh, int64_t v_sl, int64_t v_sp, int64_t v_ss, int64_t v_sh,
                             int64_t c_sl, int64_t c_sp, int64_t c_ss, int64_t c_sh, int32_t dtype,
                             void* stream) {
  ZP_REQUIRE(score_cache, "compress_kv_and_score: null score cache");
  bool fused = false;
  int rc = compress_kv_impl(key, value, flag, block_table, target_block_table, L, B, NB, BS, Hkv, D,
                            num_pages, target_width, k_sl, k_sp, k_ss, k_sh, v_sl, v_sp, v_ss, v_sh,
                            dtype, score_cache, scores_src, c_sl, c_sp, c_ss, c_sh, &fused, stream);
  if (rc != ZP_OK || fused) return rc;
  return zp_compress_score(score_cache, scores_src, flag, block_table, target_block_table, L, B, NB,
                           BS, Hkv, num_pages, target_width, c_sl, c_sp, c_ss, c_sh, dtype, stream);
}

extern "C" int zp_compress_score(void* score_cache, const void* scores_src, const uint8_t* flag,
                                 const int32_t* block_table, const int32_t* target_block_table,
                                 int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                                 int32_t num_pages, int32_t target_width, int64_t c_sl,
                                 int64_t c_sp, int64_t c_ss, int64_t c_sh, int32_t dtype,
                                 void* stream) {
  ZP_REQUIRE(score_cache && flag && block_table && target_block_table,
             "compress_score: null pointer");
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0 && target_width > 0,
             "compress_score: bad dims");
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "compress_score: unknown dtype tag %d", dtype);
  ZP_REQUIRE((int64_t)NB * BS <= 65536, "compress_score: NB*BS=%lld exceeds 65536",
             (long long)NB * BS);
  ZP_REQUIRE((int64_t)L * B * Hkv < ((int64_t)1 << 31), "compress_score: too many (layer, sequence, head) rows");
  if (L == 0 || B == 0) return ZP_OK;
  const int es = zp_dtype_bytes(dtype);
  CompactArgs a;
  a.a = (char*)score_cache; a.b = nullptr; a.flag = flag; a.table = block_table;
  a.target = target_block_table; a.rows = (const char*)scores_src;
  a.B = B; a.NB = NB; a.BS = BS; a.Hkv = Hkv; a.num_pages = num_pages;
  a.target_width = target_width; a.lpv = 1;
  a.a_sl = c_sl * es; a.a_sp = c_sp * es; a.a_ss = c_ss * es; a.a_sh = c_sh * es;
  a.b_sl = a.b_sp = a.b_ss = a.b_sh = 0;
  a.c = nullptr; a.c_rows = nullptr; a.c_sl = a.c_sp = a.c_ss = a.c_sh = 0;
  a.split_kv = 0;
  hipStream_t st = (hipStream_t)stream;
  if (es == 4) return launch_compact<uint32_t, 4, false>(a, L, st);
  return launch_compact<uint16_t, 4, false>(a, L, st);
}

extern "C" int zp_store_query(const void* query, void* query_cache, const int32_t* slot_mapping,
                              int32_t n, int32_t row_elems, int32_t num_tokens, int32_t max_seqs,
                              int32_t window, int64_t q_stride_tok, int64_t c_stride_seq,
                              int64_t c_stride_slot, int64_t sm_stride_row, int64_t sm_stride_col,
                              int32_t dtype, void* stream) {
  ZP_REQUIRE(n >= 0 && row_elems > 0, "store_query: bad dims n=%d row_elems=%d", n, row_elems);
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "store_query: unknown dtype tag %d", dtype);
  if (n == 0) return ZP_OK;
  ZP_REQUIRE(query && query_cache && slot_mapping, "store_query: null pointer");
  const int es = zp_dtype_bytes(dtype);
  const int64_t row = (int64_t)row_elems * es;
  const int64_t qs = q_stride_tok * es, cs = c_stride_seq * es, cl = c_stride_slot * es;
  int piece = 2;
  for (int cand : {16, 8, 4}) {
    if (aligned_to(row, cand) && aligned_to(qs, cand) && aligned_to(cs, cand) &&
        aligned_to(cl, cand) && aligned_to((int64_t)(uintptr_t)query, cand) &&
        aligned_to((int64_t)(uintptr_t)query_cache, cand)) {
      piece = cand;
      break;
    }
  }
  hipStream_t st = (hipStream_t)stream;
  const int pieces = (int)(row / piece);
#define ZP_SQ(P)                                                                              \
  hipLaunchKernelGGL((store_query_kernel<P>), dim3(n), dim3(kThreads), 0, st,                 \
                     (const char*)query, (char*)query_cache, slot_mapping, pieces, num_tokens, \
                     max_seqs, window, qs, cs, cl, sm_stride_row, sm_stride_col)
  switch (piece) {
    case 16: ZP_SQ(u32x4); break;
    case 8:  ZP_SQ(u32x2); break;
    case 4:  ZP_SQ(uint32_t); break;
    default: ZP_SQ(uint16_t); break;
  }
#undef ZP_SQ
  ZP_LAUNCH_CHECK();
  return ZP_OK;
}
