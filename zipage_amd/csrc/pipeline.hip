// One layer chunk of the compression step as ONE host call: the body of
// ModelRunner.compress (zipage/engine/model_runner.py:466-622) enqueued stage by stage on the
// caller's stream, with every intermediate (scores, redundancy, keep flags, kernel scratch) in a
// workspace the caller passes in.  Nothing here launches a kernel of its own: each stage is the
// entry point that also stands alone in this ABI, so results are bit-identical to calling them
// one after the other.
//
// zp_compress_layers_static is the same call for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops): its workspace is a fixed array in device
// memory that belongs to the library.
#include "common.h"

#include <mutex>

namespace {

constexpr int64_t kAlign = 256;
inline int64_t align_up(int64_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

struct Plan {
  int64_t scores, scores2, red, flag, score_ws, raw_ws, total;   // byte offsets; -1 = unused
  int64_t score_ws_bytes, raw_ws_bytes;
  bool one_launch_select;
};

// Rows the one-launch selection holds in LDS (zp_select_topk's own limit).
inline bool select_fits(int64_t Tn) { return Tn * 8 <= 150 * 1024; }

// lean: give the scorer only the scratch it cannot do without (it then sweeps K three times
// instead of keeping the logits in registers) -- for callers with a fixed scratch budget.
Plan make_plan(int L, int B, int NB, int BS, int Hkv, int Hq, int W, int dtype,
               const zp_compress_config* c, bool own_flag, bool lean = false) {
  Plan p;
  const int64_t n = (int64_t)L * B * Hkv * NB * BS;
  const int64_t es = zp_dtype_bytes(dtype);
  int64_t off = 0;
  auto take = [&](int64_t bytes) { const int64_t o = off; off += align_up(bytes); return o; };
  p.one_launch_select = select_fits((int64_t)NB * BS);
  p.scores = take(n * es);
  // the separate stages: pooling needs distinct in / out buffers, and the mask epilogue works in
  // place, which must not touch the scores the carried-score compaction reads later
  p.scores2 = (!p.one_launch_select &&
               (c->pooling_size > 1 || (c->use_global_score && c->deterministic_carry)))
                  ? take(n * es) : -1;
  p.red = c->use_redundancy ? take(n * es) : -1;
  p.flag = own_flag ? take(n) : -1;
  p.score_ws_bytes = lean ? zp_attention_score_workspace_floor(L, B, NB, BS, Hkv, Hq, W)
                          : zp_attention_score_workspace_for(L, B, NB, BS, Hkv, Hq, W, dtype);
  p.score_ws = p.score_ws_bytes ? take(p.score_ws_bytes) : -1;
  p.raw_ws_bytes = (c->use_redundancy && !c->lightning) ? zp_redundancy_raw_workspace(L, B, NB, BS, Hkv) : 0;
  p.raw_ws = p.raw_ws_bytes ? take(p.raw_ws_bytes) : -1;
  p.total = off;
  return p;
}

// Everything a stage would refuse is refused here, before the first launch: a chunk either runs
// all of its stages or none (the global-score stage rewrites the score cache when
// deterministic_carry is off, so a failure behind it would leave a half-applied step).
int check_chunk(const zp_compress_config* c, int L, int B, int NB, int BS, int Hkv, int Hq, int D,
                int W, int target_width, int dtype, bool one_launch_select, const void* score_cache) {
  ZP_REQUIRE(c, "compress_layers: null config");
  ZP_REQUIRE(L >= 0 && B >= 0 && NB > 0 && BS > 0 && Hkv > 0 && Hq > 0 && D > 0 && W > 0 &&
                 W <= BS && target_width > 0, "compress_layers: bad dims");
  ZP_REQUIRE(dtype >= ZP_BF16 && dtype <= ZP_F32, "compress_layers: unknown dtype tag %d", dtype);
  ZP_REQUIRE(Hq % Hkv == 0, "compress_layers: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  ZP_REQUIRE(c->budget_blocks > 0, "compress_layers: budget_blocks=%d", c->budget_blocks);
  ZP_REQUIRE(c->query_cache_len > 0 && c->query_cache_len <= BS,
             "compress_layers: query_cache_len=%d outside (0, BS=%d]", c->query_cache_len, BS);
  ZP_REQUIRE(c->budget_blocks <= NB, "compress_layers: keeping %d pages of a table of %d",
             c->budget_blocks, NB);
  ZP_REQUIRE(target_width >= c->budget_blocks, "compress_layers: target table of %d pages for a "
             "budget of %d", target_width, c->budget_blocks);
  ZP_REQUIRE(c->reduced == ZP_REDUCE_MEAN || c->reduced == ZP_REDUCE_MAX,
             "compress_layers: unknown reduction %d", c->reduced);
  ZP_REQUIRE(c->pooling_size >= 0 && (c->pooling_size <= 1 || (c->pooling_size & 1)),
             "compress_layers: pooling_size %d must be odd (or 0 / 1 for none)", c->pooling_size);
  ZP_REQUIRE(c->pooling_mode == ZP_POOL_MAX || c->pooling_mode == ZP_POOL_AVG,
             "compress_layers: unknown pooling mode %d", c->pooling_mode);
  ZP_REQUIRE(c->sink_len >= 0, "compress_layers: negative sink_len");
  if (c->use_global_score) {
    ZP_REQUIRE(score_cache, "compress_layers: use_global_score needs a score cache");
    ZP_REQUIRE(c->decay_factor >= 0.f && c->decay_factor <= 1.f,
               "compress_layers: decay_factor %g outside [0,1]", (double)c->decay_factor);
    ZP_REQUIRE(c->activate_method == ZP_ACTIVATE_MAX || c->activate_method == ZP_ACTIVATE_SUM,
               "compress_layers: unknown activate_method %d", c->activate_method);
  }
  const int es = zp_dtype_bytes(dtype);
  const int64_t Tn = (int64_t)NB * BS;
  if (D > 128 || (D * es) % 16 != 0) {
    zp_set_error("compress_layers: head_dim %d unsupported (need <= 128 and a multiple of %d)", D, 16 / es);
    return ZP_EUNSUPPORTED;
  }
  const int tile = es == 4 ? 64 : 128;
  if (BS % tile != 0) {
    zp_set_error("compress_layers: page size %d is not a multiple of %d", BS, tile);
    return ZP_EUNSUPPORTED;
  }
  int gp = 1;
  while (gp < Hq / Hkv) gp <<= 1;
  if (gp > 32) {
    zp_set_error("compress_layers: GQA group %d unsupported (max 32)", Hq / Hkv);
    return ZP_EUNSUPPORTED;
  }
  ZP_REQUIRE(Tn <= 65536, "compress_layers: NB*BS=%lld exceeds 65536", (long long)Tn);
  ZP_REQUIRE((int64_t)L * B * Hkv < ((int64_t)1 << 28), "compress_layers: too many (layer, sequence, head) rows");
  if (!one_launch_select && Tn * 4 > 150 * 1024) {
    zp_set_error("compress_layers: a row of %lld tokens exceeds what top-k holds in LDS", (long long)Tn);
    return ZP_EUNSUPPORTED;
  }
  if (c->use_redundancy && Tn * (c->lightning ? 4 : 12) > 150 * 1024) {
    zp_set_error("compress_layers: a row of %lld tokens exceeds what the redundancy softmax holds in LDS",
                 (long long)Tn);
    return ZP_EUNSUPPORTED;
  }
  return ZP_OK;
}

struct Stamp {
  void* const* ev;
  hipStream_t st;
  void start(int stage) const {
    if (ev && ev[2 * stage]) (void)hipEventRecord((hipEvent_t)ev[2 * stage], st);
  }
  void stop(int stage) const {
    if (ev && ev[2 * stage + 1]) (void)hipEventRecord((hipEvent_t)ev[2 * stage + 1], st);
  }
};

int run_layers(void* k_cache, void* v_cache, const void* query_cache, void* score_cache,
               const int32_t* seq_idx, const int32_t* block_table, const uint8_t* compressed,
               const int32_t* target, uint8_t* flag_out, int L, int B, int NB, int BS, int Hkv,
               int Hq, int D, int W, int num_pages, int max_seqs, int target_width,
               const int64_t* st_, int dtype, const zp_compress_config* c, char* ws,
               const Plan& p, void* const* stage_events, void* stream) {
  // strides (elements): k layer/page/slot/head, v layer/page/slot/head, q layer/seq,
  // score-cache layer/page/slot/head
  const int64_t k_sl = st_[0], k_sp = st_[1], k_ss = st_[2], k_sh = st_[3];
  const int64_t v_sl = st_[4], v_sp = st_[5], v_ss = st_[6], v_sh = st_[7];
  const int64_t q_sl = st_[8], q_ss = st_[9];
  const int64_t c_sl = st_[10], c_sp = st_[11], c_ss = st_[12], c_sh = st_[13];
  ZP_REQUIRE(k_ss == (int64_t)Hkv * D && k_sh == D,
             "compress_layers: the key cache must be contiguous in its (slot, head, dim) axes");
  const Stamp t{stage_events, (hipStream_t)stream};
  void* scores = ws + p.scores;
  void* red = p.red >= 0 ? ws + p.red : nullptr;
  uint8_t* flag = flag_out ? flag_out : (uint8_t*)(ws + p.flag);
  const float scale = c->softmax_scale > 0.f ? c->softmax_scale : 1.0f / sqrtf((float)D);
  const int k_keep = BS * c->budget_blocks;
  const bool glob = c->use_global_score != 0;
  const int max_norm_red = (c->use_redundancy && glob && c->max_norm) ? 1 : 0;
  int rc;

  t.start(ZP_STAGE_ATTENTION_SCORE);
  rc = zp_attention_score(k_cache, query_cache, seq_idx, block_table, scores, nullptr, L, B, NB,
                          BS, Hkv, Hq, D, W, num_pages, max_seqs, k_sl, k_sp, q_sl, q_ss, scale,
                          c->reduced, dtype, p.score_ws >= 0 ? ws + p.score_ws : nullptr,
                          p.score_ws_bytes, stream);
  if (rc != ZP_OK) return rc;
  t.stop(ZP_STAGE_ATTENTION_SCORE);

  if (glob) {
    ZP_REQUIRE(score_cache, "compress_layers: use_global_score needs a score cache");
    ZP_REQUIRE(c_ss == Hkv && c_sh == 1, "compress_layers: score cache must be (slot, head) contiguous");
    t.start(ZP_STAGE_GLOBAL_SCORE);
    if (c->max_norm) {
      rc = zp_score_epilogue(scores, nullptr, block_table, L, B, NB, BS, Hkv, 1, 0, 0.0, 0, 0, 0,
                             dtype, stream);
      if (rc != ZP_OK) return rc;
    }
    rc = zp_global_score(scores, score_cache, block_table, compressed, L, B, NB, BS, Hkv,
                         num_pages, c_sl, c_sp, c->decay_factor, c->activate_method,
                         c->deterministic_carry ? 0 : 1, dtype, stream);
    if (rc != ZP_OK) return rc;
    t.stop(ZP_STAGE_GLOBAL_SCORE);
  }

  if (c->use_redundancy) {
    t.start(ZP_STAGE_REDUNDANCY);
    if (c->lightning)
      rc = zp_redundancy_lightning(k_cache, block_table, red, nullptr, L, B, NB, BS, Hkv, D,
                                   num_pages, k_sl, k_sp, c->redundancy_threshold,
                                   c->redundancy_temperature, dtype, stream);
    else
      rc = zp_redundancy_raw(k_cache, block_table, red, nullptr, L, B, NB, BS, Hkv, D, num_pages,
                             k_sl, k_sp, c->redundancy_threshold, c->redundancy_temperature, dtype,
                             ws + p.raw_ws, p.raw_ws_bytes, stream);
    if (rc != ZP_OK) return rc;
    t.stop(ZP_STAGE_REDUNDANCY);
  }

  // what the compaction of the carried scores reads in the deterministic mode: the scores as
  // zp_global_score left them
  const void* carried = (glob && c->deterministic_carry) ? scores : nullptr;
  if (p.one_launch_select) {
    t.start(ZP_STAGE_SELECT);
    rc = zp_select_topk(scores, nullptr, red, flag, block_table, compressed, L, B, NB, BS, Hkv,
                        c->pooling_size, c->continues_pooling, c->pooling_mode, max_norm_red,
                        c->redundancy_lambda, c->sink_len, c->query_cache_len, 1, k_keep, dtype,
                        stream);
    if (rc != ZP_OK) return rc;
    t.stop(ZP_STAGE_SELECT);
  } else {
    // rows too long for the one-launch selection: the reference's separate stages
    void* cur = scores;
    if (c->pooling_size <= 1 && p.scores2 >= 0) {
      cur = ws + p.scores2;
      if (hipMemcpyAsync(cur, scores, (size_t)L * B * Hkv * NB * BS * zp_dtype_bytes(dtype),
                         hipMemcpyDeviceToDevice, (hipStream_t)stream) != hipSuccess) {
        zp_set_error("compress_layers: device copy of the scores failed");
        return ZP_EHIP;
      }
    }
    if (c->pooling_size > 1) {
      t.start(ZP_STAGE_POOLING);
      rc = zp_pool_scores(scores, ws + p.scores2, compressed, L, B, Hkv, NB * BS, c->pooling_size,
                          c->continues_pooling, c->pooling_mode, dtype, stream);
      if (rc != ZP_OK) return rc;
      cur = ws + p.scores2;
      t.stop(ZP_STAGE_POOLING);
    }
    t.start(ZP_STAGE_WINDOW_MASK);
    rc = zp_score_epilogue(cur, red, block_table, L, B, NB, BS, Hkv, 0, max_norm_red,
                           c->redundancy_lambda, c->sink_len, c->query_cache_len, 1, dtype, stream);
    if (rc != ZP_OK) return rc;
    t.stop(ZP_STAGE_WINDOW_MASK);
    t.start(ZP_STAGE_TOPK_MASK);
    ZP_REQUIRE((int64_t)L * B * Hkv < ((int64_t)1 << 31), "compress_layers: too many rows");
    rc = zp_topk_mask(cur, flag, L * B * Hkv, NB * BS, k_keep, dtype, stream);
    if (rc != ZP_OK) return rc;
    t.stop(ZP_STAGE_TOPK_MASK);
  }

  // with a carried score cache the scores of the survivors move in the K/V launch (the stage events
  // of the score compaction are then recorded back to back: its time is inside compress_kv)
  t.start(ZP_STAGE_COMPRESS_KV);
  if (glob)
    rc = zp_compress_kv_and_score(k_cache, v_cache, score_cache, carried, flag, block_table, target, L,
                                  B, NB, BS, Hkv, D, num_pages, target_width, k_sl, k_sp, k_ss, k_sh,
                                  v_sl, v_sp, v_ss, v_sh, c_sl, c_sp, c_ss, c_sh, dtype, stream);
  else
    rc = zp_compress_kv(k_cache, v_cache, flag, block_table, target, L, B, NB, BS, Hkv, D,
                        num_pages, target_width, k_sl, k_sp, k_ss, k_sh, v_sl, v_sp, v_ss, v_sh,
                        dtype, stream);
  if (rc != ZP_OK) return rc;
  t.stop(ZP_STAGE_COMPRESS_KV);
  if (glob) {
    t.start(ZP_STAGE_COMPRESS_SCORE);
    t.stop(ZP_STAGE_COMPRESS_SCORE);
  }
  return ZP_OK;
}

// ---- the library's own scratch: one array per GPU, in that GPU's memory, for the life of the
// process.  Host code only ever uses the address hipGetSymbolAddress returns for it.
static __device__ __align__(256) unsigned char scratch[ZP_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
char* g_scratch_ptr[kMaxDevices] = {nullptr};

int static_scratch(char** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    zp_set_error("compress_layers_static: no current device (%s)", hipGetErrorString(e));
    return ZP_EHIP;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      zp_set_error("compress_layers_static: hipGetSymbolAddress failed on device %d: %s", dev,
                   hipGetErrorString(e));
      return ZP_EHIP;
    }
    g_scratch_ptr[dev] = (char*)ptr;
  }
  *out = g_scratch_ptr[dev];
  return ZP_OK;
}

}  // namespace

extern "C" int zp_static_scratch_init(void) {
  char* ws = nullptr;
  return static_scratch(&ws);
}

extern "C" int64_t zp_compress_layers_workspace(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                                int32_t Hkv, int32_t Hq, int32_t W, int32_t dtype,
                                                const zp_compress_config* cfg,
                                                int32_t flag_in_workspace) {
  if (!cfg || L < 0 || B < 0 || NB <= 0 || BS <= 0 || Hkv <= 0 || Hq <= 0 || W <= 0 ||
      dtype < ZP_BF16 || dtype > ZP_F32)
    return -1;
  return make_plan(L, B, NB, BS, Hkv, Hq, W, dtype, cfg, flag_in_workspace != 0).total;
}

extern "C" int zp_compress_layers(void* k_cache, void* v_cache, const void* query_cache,
                                  void* score_cache, const int32_t* seq_idx,
                                  const int32_t* block_table, const uint8_t* compressed,
                                  const int32_t* target_block_table, uint8_t* flag_out,
                                  int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                                  int32_t Hq, int32_t D, int32_t W, int32_t num_pages,
                                  int32_t max_seqs, int32_t target_width, const int64_t* strides,
                                  int32_t dtype, const zp_compress_config* cfg, void* workspace,
                                  int64_t workspace_bytes, void* const* stage_events,
                                  void* stream) {
  ZP_REQUIRE(cfg, "compress_layers: null config");
  int rc = check_chunk(cfg, L, B, NB, BS, Hkv, Hq, D, W, target_width, dtype,
                       select_fits((int64_t)NB * BS), score_cache);
  if (rc != ZP_OK) return rc;
  ZP_REQUIRE(k_cache && v_cache && query_cache && seq_idx && block_table && compressed &&
                 target_block_table && strides, "compress_layers: null pointer");
  if (L == 0 || B == 0) return ZP_OK;
  const Plan p = make_plan(L, B, NB, BS, Hkv, Hq, W, dtype, cfg, flag_out == nullptr);
  ZP_REQUIRE(workspace && workspace_bytes >= p.total,
             "compress_layers: workspace of %lld bytes required, %lld given", (long long)p.total,
             (long long)workspace_bytes);
  ZP_REQUIRE(((uintptr_t)workspace % kAlign) == 0, "compress_layers: workspace must be 256-byte aligned");
  return run_layers(k_cache, v_cache, query_cache, score_cache, seq_idx, block_table, compressed,
                    target_block_table, flag_out, L, B, NB, BS, Hkv, Hq, D, W, num_pages, max_seqs,
                    target_width, strides, dtype, cfg, (char*)workspace, p, stage_events, stream);
}

extern "C" int zp_compress_layers_static(void* k_cache, void* v_cache, const void* query_cache,
                                         void* score_cache, const int32_t* seq_idx,
                                         const int32_t* block_table, const uint8_t* compressed,
                                         const int32_t* target_block_table, uint8_t* flag_out,
                                         int32_t L, int32_t B, int32_t NB, int32_t BS,
                                         int32_t Hkv, int32_t Hq, int32_t D, int32_t W,
                                         int32_t num_pages, int32_t max_seqs,
                                         int32_t target_width, const int64_t* strides,
                                         int32_t dtype, const zp_compress_config* cfg,
                                         void* stream) {
  ZP_REQUIRE(cfg, "compress_layers_static: null config");
  int rc = check_chunk(cfg, L, B, NB, BS, Hkv, Hq, D, W, target_width, dtype,
                       select_fits((int64_t)NB * BS), score_cache);
  if (rc != ZP_OK) return rc;
  ZP_REQUIRE(k_cache && v_cache && query_cache && seq_idx && block_table && compressed &&
                 target_block_table && strides, "compress_layers_static: null pointer");
  if (L == 0 || B == 0) return ZP_OK;
  Plan p = make_plan(L, B, NB, BS, Hkv, Hq, W, dtype, cfg, flag_out == nullptr);
  if (p.total > (int64_t)ZP_STATIC_SCRATCH_BYTES)
    p = make_plan(L, B, NB, BS, Hkv, Hq, W, dtype, cfg, flag_out == nullptr, true);
  ZP_REQUIRE(p.total <= (int64_t)ZP_STATIC_SCRATCH_BYTES,
             "compress_layers_static: this chunk needs %lld bytes of scratch, the library's array "
             "holds %lld; split the batch or the layers, or use zp_compress_layers with a "
             "workspace", (long long)p.total, (long long)ZP_STATIC_SCRATCH_BYTES);
  char* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != ZP_OK) return rc;
  return run_layers(k_cache, v_cache, query_cache, score_cache, seq_idx, block_table, compressed,
                    target_block_table, flag_out, L, B, NB, BS, Hkv, Hq, D, W, num_pages, max_seqs,
                    target_width, strides, dtype, cfg, ws, p, nullptr, stream);
}
