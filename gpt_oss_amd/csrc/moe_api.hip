// Host side of the C-ABI (include/moe_abi.h): handle, weight ingest, stage
// orchestration, per-stage event timing.  Plays the role of the host code of
// getp-csrc/expert.cpp (init :709-1174, forward :1366-1607, cleanup :1234-1364)
// and of the local MoE path in getp_run.cpp:697-845, for one GPU.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <new>
#include <vector>

#include "moe_internal.h"

using namespace moe;

namespace {
thread_local char g_err[512] = "";
}

// Records the text of a failure for moe_last_error() and returns `code`.
int moe::set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

namespace {

#define fail moe::set_error

#define HIP_TRY(call)                                                                       \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      return fail(MOE_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, \
                  __LINE__);                                                                \
  } while (0)

int next_router_pad(int E) {
  for (int p = 16; p <= 256; p <<= 1)
    if (E <= p) return p;
  return -1;
}

constexpr int kMaxProfileCalls = 256;

}  // namespace

struct moe_handle {
  moe_config cfg{};
  int device = 0;
  int E_pad = 0;
  int Hp = 0, IMp = 0;  // hidden / inter as the GEMMs see them: padded to multiples of 64
  std::vector<LayerWeights> layers;
  size_t layer_bytes = 0;
  size_t ws_bytes = 0;

  // routing produced by the router stage (or copied from the caller)
  int *topk_i = nullptr;
  float *topk_v = nullptr;
  // dispatch
  DispatchBuffers disp{};
  int a_cap = 0;      // max assignments
  int a_pad_cap = 0;  // max padded rows
  int n_blk_cap = 0;
  int disp_tokens = -1;  // batch of the last moe_dispatch (stage-level calls), -1: none
  bool gemms_done = false;  // moe_expert_gemms has run on that dispatch: y holds its rows
  bool distinct_ids = false;  // moe_set_distinct_ids: caller-supplied ids name an expert once per token
  // The last call ran without a dispatch pass (at most 64 tokens): its ids, for a
  // moe_get_dispatch that asks for the plan afterwards.  topk_i == nullptr: none.
  DirectIds unplanned{nullptr, nullptr, 0, 0};
  // expert pipeline
  uint16_t *act = nullptr;  // SwiGLU output, bf16 fragments
  float *y = nullptr;       // down output [a_pad_cap, Hp], then the second part of a split reduction
  int y_parts = 1;          // copies of y the last down GEMM wrote (down_k_split)
  uint16_t *t_norm = nullptr;  // normalised rows of moe_block_forward [max_tokens, H], allocated on first use
  uint16_t *x_pad = nullptr;   // the batch's rows widened to Hp columns [max_tokens, Hp]; only where Hp != H

  // profiling
  std::vector<hipEvent_t> events;  // kMaxProfileCalls * (MOE_NUM_STAGES + 1)
  int prof_armed = 0;              // calls still to record
  int prof_recorded = 0;
};

namespace {

template <typename T>
int dev_alloc(moe_handle *h, T **p, size_t count, bool workspace) {
  void *q = nullptr;
  const size_t bytes = count * sizeof(T);
  hipError_t e = hipMalloc(&q, bytes ? bytes : 1);
  if (e != hipSuccess)
    return fail(MOE_ERR_HIP, "hipMalloc(%zu bytes) failed: %s", bytes, hipGetErrorString(e));
  *p = static_cast<T *>(q);
  if (workspace) h->ws_bytes += bytes;
  return MOE_OK;
}

int check_forward_args(moe_handle *h, int layer, const void *x, int n_tokens, const void *out) {
  if (!h) return fail(MOE_ERR_BAD_ARG, "null handle");
  if (layer < 0 || layer >= h->cfg.layers)
    return fail(MOE_ERR_BAD_ARG, "layer %d out of range [0,%d)", layer, h->cfg.layers);
  if (n_tokens < 0) return fail(MOE_ERR_BAD_ARG, "n_tokens %d is negative", n_tokens);
  if (n_tokens > h->cfg.max_tokens)
    return fail(MOE_ERR_CAPACITY, "n_tokens %d exceeds max_tokens %d", n_tokens, h->cfg.max_tokens);
  if (n_tokens > 0 && (!x || !out)) return fail(MOE_ERR_BAD_ARG, "null device pointer");
  // the kernels read the rows of x in 16-byte pieces (a row is a multiple of 128 bytes)
  if ((reinterpret_cast<uintptr_t>(x) & 15) != 0)
    return fail(MOE_ERR_BAD_ARG, "x is not 16-byte aligned");
  if (!h->layers[layer].uploaded)
    return fail(MOE_ERR_STATE, "layer %d has no weights (moe_upload_layer not called)", layer);
  return MOE_OK;
}

struct StageTimer {
  moe_handle *h;
  hipStream_t s;
  hipEvent_t *ev = nullptr;
  StageTimer(moe_handle *h_, hipStream_t s_) : h(h_), s(s_) {
    if (h->prof_armed > 0 && h->prof_recorded < kMaxProfileCalls && !h->events.empty())
      ev = &h->events[(size_t)h->prof_recorded * (MOE_NUM_STAGES + 1)];
  }
  hipError_t mark(int boundary) {  // boundary i = start of stage i; MOE_NUM_STAGES = end
    return ev ? hipEventRecord(ev[boundary], s) : hipSuccess;
  }
  void done() {
    if (ev) {
      h->prof_recorded++;
      h->prof_armed--;
    }
  }
};

// column tiles of the two grouped GEMMs (tiles are kGemmTileNb blocks of 32 columns wide)
inline int gate_up_col_tiles(const moe_handle *h) {
  return (2 * h->IMp / kRowBlock + kGemmTileNb - 1) / kGemmTileNb;
}
inline int down_col_tiles(const moe_handle *h) {
  return (h->Hp / kRowBlock + kGemmTileNb - 1) / kGemmTileNb;
}

// Stages 3-4 on the plan of the last dispatch: gate_up GEMM with the SwiGLU (it
// reads the routed token rows itself, there is no gathered copy), down GEMM.
// Leaves the per-assignment rows in h->y.
// max_rows: no expert is given more rows than this (T when the ids of a token are distinct).
int run_gemms(moe_handle *h, int layer, const uint16_t *x, int T, int max_rows, const DirectIds &direct,
              hipStream_t s, StageTimer &tm) {
  const moe_config &c = h->cfg;
  const LayerWeights &lw = h->layers[layer];
  const int A = T * kTopK;
  const int mt_cap = A / kTileRows + c.experts;
  HIP_TRY(tm.mark(MOE_STAGE_GATE_UP));
  if (h->Hp != c.hidden) {  // a hidden size that is not a multiple of 64: rows widened with zeros
    HIP_TRY(launch_pad_rows(x, h->x_pad, T, c.hidden, h->Hp, s));
    x = h->x_pad;
  }
  HIP_TRY(launch_gate_up(x, lw.w1q ? static_cast<const void *>(lw.w1q) : lw.w1, lw.w1s, lw.b1g, lw.b1u,
                         h->disp, h->act, h->Hp, h->IMp, c.swiglu_limit, mt_cap, max_rows, direct, s));
  HIP_TRY(tm.mark(MOE_STAGE_DOWN));
  HIP_TRY(launch_down(h->act, lw.w2q ? static_cast<const void *>(lw.w2q) : lw.w2, lw.w2s, lw.b2,
                      h->disp, h->y, h->Hp, h->IMp, mt_cap, max_rows, direct,
                      down_k_split(max_rows, h->IMp, h->Hp, c.experts, T),
                      (size_t)h->a_pad_cap * h->Hp * sizeof(float), s));
  h->y_parts = down_k_split(max_rows, h->IMp, h->Hp, c.experts, T);
  return MOE_OK;
}

// Stage 6: out != nullptr: out (+)= sum_k w[t,k] * y[row of (t,k)], fp32.
// Otherwise resid (bf16, in place) += that sum.
int run_combine(moe_handle *h, const float *topk_v, const int *pos, int T, float *out, int accumulate,
                uint16_t *resid, const DirectIds &direct, hipStream_t s, StageTimer &tm) {
  HIP_TRY(tm.mark(MOE_STAGE_COMBINE));
  if (out) {
    HIP_TRY(launch_combine(h->y, h->Hp, h->y_parts, (size_t)h->a_pad_cap * h->Hp, h->disp.inv, topk_v, pos, out, T,
                           h->cfg.hidden, accumulate, direct, s));
  } else {
    HIP_TRY(launch_combine_residual(h->y, h->Hp, h->y_parts, (size_t)h->a_pad_cap * h->Hp, h->disp.inv, topk_v, pos,
                                    resid, T, h->cfg.hidden, direct, s));
  }
  HIP_TRY(tm.mark(MOE_NUM_STAGES));
  return MOE_OK;
}

// Stages 2-6.
int run_experts(moe_handle *h, int layer, const uint16_t *x, const int *pos, const int *topk_i,
                const float *topk_v, int T, int max_rows, float *out, int accumulate, hipStream_t s,
                StageTimer &tm, uint16_t *resid = nullptr) {
  const moe_config &c = h->cfg;
  HIP_TRY(tm.mark(MOE_STAGE_DISPATCH));
  // a batch of at most 64 tokens needs no dispatch pass: the GEMMs and the
  // combine find their rows from the ids themselves
  const bool direct_plan = direct_plan_fits(T, max_rows, c.experts, h->a_pad_cap);
  const DirectIds direct{direct_plan ? topk_i : nullptr, pos, T, c.experts};
  if (!direct_plan)
    HIP_TRY(launch_dispatch(topk_i, pos, T, c.experts, gate_up_col_tiles(h), down_col_tiles(h), h->disp, s));
  h->unplanned = direct;
  h->disp_tokens = -1;  // the plan now belongs to this call, not to a moe_dispatch
  h->gemms_done = false;
  int rc = run_gemms(h, layer, x, T, max_rows, direct, s, tm);
  if (rc != MOE_OK) return rc;
  return run_combine(h, topk_v, pos, T, out, accumulate, resid, direct, s, tm);
}

}  // namespace

extern "C" {

const char *moe_last_error(void) { return g_err; }
const char *moe_version(void) { return "mi355-moe 0.1 (gfx950)"; }

int moe_create(const moe_config *cfg, moe_handle **out) {
  if (!cfg || !out) return fail(MOE_ERR_BAD_ARG, "null argument");
  *out = nullptr;
  if (cfg->topk != kTopK)
    return fail(MOE_ERR_UNSUPPORTED, "topk %d unsupported (kernels are built for 4)", cfg->topk);
  if (cfg->hidden <= 0 || cfg->hidden % 32 || cfg->inter <= 0 || cfg->inter % 32)
    return fail(MOE_ERR_UNSUPPORTED, "hidden %d / inter %d must be positive multiples of 32",
                cfg->hidden, cfg->inter);
  if (cfg->experts < kTopK || cfg->experts > 256)
    return fail(MOE_ERR_UNSUPPORTED, "experts %d outside [4,256]", cfg->experts);
  if (cfg->layers <= 0 || cfg->max_tokens <= 0)
    return fail(MOE_ERR_BAD_ARG, "layers %d / max_tokens %d must be positive", cfg->layers,
                cfg->max_tokens);
  if ((long long)cfg->max_tokens * kTopK > (1ll << 28))
    return fail(MOE_ERR_UNSUPPORTED, "max_tokens %d too large", cfg->max_tokens);
  if (!(cfg->swiglu_limit > 0.f)) return fail(MOE_ERR_BAD_ARG, "swiglu_limit must be positive");

  moe_handle *h = new (std::nothrow) moe_handle();
  if (!h) return fail(MOE_ERR_BAD_ARG, "out of host memory");
  h->cfg = *cfg;
  h->E_pad = next_router_pad(cfg->experts);
  h->Hp = padded_dim(cfg->hidden);
  h->IMp = padded_dim(cfg->inter);
  hipError_t e = hipGetDevice(&h->device);
  if (e != hipSuccess) {
    delete h;
    return fail(MOE_ERR_HIP, "hipGetDevice failed: %s", hipGetErrorString(e));
  }
  h->layers.resize(cfg->layers);

  const int E = cfg->experts, H = cfg->hidden, IM = cfg->inter, T = cfg->max_tokens;
  h->a_cap = T * kTopK;
  h->a_pad_cap = ((h->a_cap + kTileGran * E + kTileGran - 1) / kTileGran) * kTileGran;
  // room for the fixed slots of the batches that run without a dispatch pass
  if (h->a_pad_cap < kDirectSlotRows * E) h->a_pad_cap = kDirectSlotRows * E;
  h->n_blk_cap = (T + 255) / 256;
  int rc = MOE_OK;
#define ALLOC(ptr, count)                                   \
  if (rc == MOE_OK) rc = dev_alloc(h, &(ptr), (count), true)
  ALLOC(h->topk_i, (size_t)h->a_cap);
  ALLOC(h->topk_v, (size_t)h->a_cap);
  ALLOC(h->disp.blk_counts, (size_t)h->n_blk_cap * E);
  ALLOC(h->disp.offsets, (size_t)E + 1);
  ALLOC(h->disp.perm, (size_t)h->a_cap);
  ALLOC(h->disp.rowmap, (size_t)h->a_pad_cap);
  ALLOC(h->disp.inv, (size_t)h->a_cap);
  ALLOC(h->disp.info, (size_t)E);
  ALLOC(h->disp.totals, (size_t)kTotInts);
  {
    const int mt_cap = h->a_cap / kTileRows + E;  // row tiles at max_tokens, at most
    h->disp.tile_cap_gate_up = mt_cap * gate_up_col_tiles(h);
    h->disp.tile_cap_down = mt_cap * down_col_tiles(h);
  }
  ALLOC(h->disp.tiles_gate_up, (size_t)h->disp.tile_cap_gate_up);
  ALLOC(h->disp.tiles_down, (size_t)h->disp.tile_cap_down);
  ALLOC(h->act, (size_t)h->a_pad_cap * h->IMp);
  // behind the rows of y: the second part of a split reduction (small batches, see down_k_split)
  ALLOC(h->y, ((size_t)h->a_pad_cap + (kSmallBatchKSplit - 1) * small_batch_pad_rows(E)) * h->Hp);
  if (h->Hp != H) ALLOC(h->x_pad, (size_t)T * h->Hp);
#undef ALLOC
  h->disp.a_pad_cap = h->a_pad_cap;
  if (rc != MOE_OK) {
    moe_destroy(h);
    return rc;
  }
  h->layer_bytes = (size_t)h->E_pad * H * 2 + (size_t)h->E_pad * 4 +
                   (size_t)E * 2 * h->IMp * h->Hp * 2 + (size_t)E * 2 * h->IMp * 4 +
                   (size_t)E * h->Hp * h->IMp * 2 + (size_t)E * h->Hp * 4;
  *out = h;
  return MOE_OK;
}

int moe_destroy(moe_handle *h) {
  if (!h) return MOE_OK;
  for (auto &lw : h->layers) {
    (void)hipFree(lw.wr); (void)hipFree(lw.br); (void)hipFree(lw.w1); (void)hipFree(lw.b1g);
    (void)hipFree(lw.b1u); (void)hipFree(lw.w2); (void)hipFree(lw.b2); (void)hipFree(lw.rms_w);
    (void)hipFree(lw.w1q); (void)hipFree(lw.w1s); (void)hipFree(lw.w2q); (void)hipFree(lw.w2s);
  }
  (void)hipFree(h->topk_i); (void)hipFree(h->topk_v);
  (void)hipFree(h->disp.blk_counts); (void)hipFree(h->disp.offsets); (void)hipFree(h->disp.perm);
  (void)hipFree(h->disp.rowmap); (void)hipFree(h->disp.inv); (void)hipFree(h->disp.info); (void)hipFree(h->disp.totals);
  (void)hipFree(h->disp.tiles_gate_up); (void)hipFree(h->disp.tiles_down);
  (void)hipFree(h->act); (void)hipFree(h->y); (void)hipFree(h->t_norm); (void)hipFree(h->x_pad);
  for (hipEvent_t ev : h->events) (void)hipEventDestroy(ev);
  delete h;
  return MOE_OK;
}

namespace {

// Source of one layer's expert matrices: fp32 as the reference keeps them on
// the host, or MXFP4 blocks and scales as the checkpoints hold them.
struct ExpertSource {
  const float *w1 = nullptr, *w2 = nullptr;
  const uint8_t *w1_blocks = nullptr, *w1_scales = nullptr, *w2_blocks = nullptr, *w2_scales = nullptr;
  bool mxfp4 = false;
};

int upload_layer(moe_handle *h, int layer, const float *w_router, const float *b_router,
                 const float *b_mlp1, const float *b_mlp2, const ExpertSource &src) {
  const int E = h->cfg.experts, H = h->cfg.hidden, IM = h->cfg.inter, E_pad = h->E_pad;
  const int Hp = h->Hp, IMp = h->IMp;
  LayerWeights &lw = h->layers[layer];
  // not usable until this upload has gone through: a failure below leaves the
  // layer without weights rather than with freed or half-written ones
  lw.uploaded = false;
  int rc = MOE_OK;
#define ALLOCW(ptr, count)                                             \
  if (rc == MOE_OK && !(ptr)) rc = dev_alloc(h, &(ptr), (count), false)
  // MXFP4 sources stay MXFP4 on the device: a quarter of the bytes, and the
  // GEMMs decode them in registers.
  const bool keep_fp4 = src.mxfp4;
  const size_t n1 = (size_t)2 * IM * H, n2 = (size_t)H * IM;  // elements of one expert's matrices
  const size_t p1 = (size_t)2 * IMp * Hp, p2 = (size_t)Hp * IMp;  // ... as packed (sides padded to 64)
  // a layer uploaded again in the other format gives the old copy back
  if (keep_fp4) {
    (void)hipFree(lw.w1); (void)hipFree(lw.w2);
    lw.w1 = lw.w2 = nullptr;
  } else {
    (void)hipFree(lw.w1q); (void)hipFree(lw.w1s); (void)hipFree(lw.w2q); (void)hipFree(lw.w2s);
    lw.w1q = lw.w2q = nullptr;
    lw.w1s = lw.w2s = nullptr;
  }
  ALLOCW(lw.wr, (size_t)E_pad * H);
  ALLOCW(lw.br, (size_t)E_pad + 2);
  ALLOCW(lw.b1g, (size_t)E * IMp);
  ALLOCW(lw.b1u, (size_t)E * IMp);
  ALLOCW(lw.b2, (size_t)E * Hp);
  if (keep_fp4) {
    ALLOCW(lw.w1q, (size_t)E * p1 / 2);
    ALLOCW(lw.w1s, (size_t)E * p1 / 64);  // two scale bytes per uint16
    ALLOCW(lw.w2q, (size_t)E * p2 / 2);
    ALLOCW(lw.w2s, (size_t)E * p2 / 64);
  } else {
    ALLOCW(lw.w1, (size_t)E * p1);
    ALLOCW(lw.w2, (size_t)E * p2);
  }
#undef ALLOCW
  if (rc != MOE_OK) return rc;

  // Staging for one expert matrix at a time; conversion and re-ordering run on
  // the GPU (the reference packs on the host, utility.cpp:568-622).
  const size_t stage_elems = (size_t)2 * IM * H > (size_t)E * H ? (size_t)2 * IM * H : (size_t)E * H;
  float *stage = nullptr, *stage_b = nullptr;
  HIP_TRY(hipMalloc(reinterpret_cast<void **>(&stage), stage_elems * sizeof(float)));
  const size_t bias_elems = (size_t)E * 2 * IM > (size_t)E * H ? (size_t)E * 2 * IM : (size_t)E * H;
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&stage_b), bias_elems * sizeof(float));
  if (e != hipSuccess) {
    (void)hipFree(stage);
    return fail(MOE_ERR_HIP, "hipMalloc failed: %s", hipGetErrorString(e));
  }
  auto body = [&]() -> int {
    HIP_TRY(hipMemcpy(stage, w_router, (size_t)E * H * sizeof(float), hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(stage_b, b_router, (size_t)E * sizeof(float), hipMemcpyHostToDevice));
    HIP_TRY(launch_pack_router(stage, stage_b, lw.wr, lw.br, E, E_pad, H, nullptr));
    HIP_TRY(launch_router_stats(stage, stage_b, E, H, lw.br + E_pad, nullptr));
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(stage_b, b_mlp1, (size_t)E * 2 * IM * sizeof(float), hipMemcpyHostToDevice));
    HIP_TRY(launch_pack_bias(stage_b, lw.b1g, lw.b1u, E, 2 * IM, 2 * IMp, true, nullptr));
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(stage_b, b_mlp2, (size_t)E * H * sizeof(float), hipMemcpyHostToDevice));
    HIP_TRY(launch_pack_bias(stage_b, lw.b2, nullptr, E, H, Hp, false, nullptr));
    HIP_TRY(hipDeviceSynchronize());
    // the staging buffer holds either an fp32 matrix or, in its place, the
    // (eight times smaller) blocks followed by the scales of an MXFP4 matrix
    uint8_t *stage_u8 = reinterpret_cast<uint8_t *>(stage);
    for (int ex = 0; ex < E; ex++) {
      if (!src.mxfp4) {
        HIP_TRY(hipMemcpy(stage, src.w1 + ex * n1, n1 * sizeof(float), hipMemcpyHostToDevice));
        HIP_TRY(launch_pack_weight(stage, lw.w1 + ex * p1, 2 * IM, H, 2 * IMp, Hp, true, nullptr));
        HIP_TRY(hipDeviceSynchronize());
        HIP_TRY(hipMemcpy(stage, src.w2 + ex * n2, n2 * sizeof(float), hipMemcpyHostToDevice));
        HIP_TRY(launch_pack_weight(stage, lw.w2 + ex * p2, H, IM, Hp, IMp, false, nullptr));
        HIP_TRY(hipDeviceSynchronize());
      } else {
        HIP_TRY(hipMemcpy(stage_u8, src.w1_blocks + ex * (n1 / 2), n1 / 2, hipMemcpyHostToDevice));
        HIP_TRY(hipMemcpy(stage_u8 + n1 / 2, src.w1_scales + ex * (n1 / 32), n1 / 32,
                          hipMemcpyHostToDevice));
        HIP_TRY(launch_pack_fp4(stage_u8, stage_u8 + n1 / 2, lw.w1q + ex * (p1 / 2),
                                lw.w1s + ex * (p1 / 64), 2 * IM, H, 2 * IMp, Hp, true, nullptr));
        HIP_TRY(hipDeviceSynchronize());
        HIP_TRY(hipMemcpy(stage_u8, src.w2_blocks + ex * (n2 / 2), n2 / 2, hipMemcpyHostToDevice));
        HIP_TRY(hipMemcpy(stage_u8 + n2 / 2, src.w2_scales + ex * (n2 / 32), n2 / 32,
                          hipMemcpyHostToDevice));
        HIP_TRY(launch_pack_fp4(stage_u8, stage_u8 + n2 / 2, lw.w2q + ex * (p2 / 2),
                                lw.w2s + ex * (p2 / 64), H, IM, Hp, IMp, false, nullptr));
        HIP_TRY(hipDeviceSynchronize());
      }
    }
    return MOE_OK;
  };
  rc = body();
  (void)hipFree(stage);
  (void)hipFree(stage_b);
  if (rc == MOE_OK) lw.uploaded = true;
  return rc;
}

int check_upload_args(moe_handle *h, int layer) {
  if (!h) return fail(MOE_ERR_BAD_ARG, "null handle");
  if (layer < 0 || layer >= h->cfg.layers)
    return fail(MOE_ERR_BAD_ARG, "layer %d out of range [0,%d)", layer, h->cfg.layers);
  return MOE_OK;
}

}  // namespace

int moe_upload_layer(moe_handle *h, int layer, const float *w_router, const float *b_router,
                     const float *w_mlp1, const float *b_mlp1, const float *w_mlp2,
                     const float *b_mlp2) {
  const int rc = check_upload_args(h, layer);
  if (rc != MOE_OK) return rc;
  if (!w_router || !b_router || !w_mlp1 || !b_mlp1 || !w_mlp2 || !b_mlp2)
    return fail(MOE_ERR_BAD_ARG, "null weight pointer");
  ExpertSource src;
  src.w1 = w_mlp1;
  src.w2 = w_mlp2;
  return upload_layer(h, layer, w_router, b_router, b_mlp1, b_mlp2, src);
}

int moe_upload_layer_mxfp4(moe_handle *h, int layer, const float *w_router, const float *b_router,
                           const uint8_t *w_mlp1_blocks, const uint8_t *w_mlp1_scales,
                           const float *b_mlp1, const uint8_t *w_mlp2_blocks,
                           const uint8_t *w_mlp2_scales, const float *b_mlp2) {
  const int rc = check_upload_args(h, layer);
  if (rc != MOE_OK) return rc;
  if (!w_router || !b_router || !w_mlp1_blocks || !w_mlp1_scales || !b_mlp1 || !w_mlp2_blocks ||
      !w_mlp2_scales || !b_mlp2)
    return fail(MOE_ERR_BAD_ARG, "null weight pointer");
  ExpertSource src;
  src.mxfp4 = true;
  src.w1_blocks = w_mlp1_blocks;
  src.w1_scales = w_mlp1_scales;
  src.w2_blocks = w_mlp2_blocks;
  src.w2_scales = w_mlp2_scales;
  return upload_layer(h, layer, w_router, b_router, b_mlp1, b_mlp2, src);
}

int moe_router(moe_handle *h, int layer, const uint16_t *x, const int *pos, int n_tokens,
               float *score, int *topk_i, float *topk_v, void *stream) {
  int rc = check_forward_args(h, layer, x, n_tokens, topk_i);
  if (rc != MOE_OK) return rc;
  if (n_tokens > 0 && !topk_v) return fail(MOE_ERR_BAD_ARG, "null device pointer");
  if (n_tokens == 0) return MOE_OK;
  const LayerWeights &lw = h->layers[layer];
  HIP_TRY(launch_router(x, pos, lw.wr, lw.br, lw.br + h->E_pad, n_tokens, h->cfg.hidden, h->cfg.experts,
                        h->E_pad, score, topk_i, topk_v, static_cast<hipStream_t>(stream)));
  return MOE_OK;
}

int moe_dispatch(moe_handle *h, const int *topk_i, const int *pos, int n_tokens, void *stream) {
  if (!h) return fail(MOE_ERR_BAD_ARG, "null handle");
  if (n_tokens < 0) return fail(MOE_ERR_BAD_ARG, "n_tokens %d is negative", n_tokens);
  if (n_tokens > h->cfg.max_tokens)
    return fail(MOE_ERR_CAPACITY, "n_tokens %d exceeds max_tokens %d", n_tokens, h->cfg.max_tokens);
  if (n_tokens > 0 && !topk_i) return fail(MOE_ERR_BAD_ARG, "null device pointer");
  HIP_TRY(launch_dispatch(topk_i, pos, n_tokens, h->cfg.experts, gate_up_col_tiles(h),
                          down_col_tiles(h), h->disp, static_cast<hipStream_t>(stream)));
  h->disp_tokens = n_tokens;
  h->gemms_done = false;
  h->unplanned.topk_i = nullptr;
  return MOE_OK;
}

int moe_get_dispatch(moe_handle *h, int *offsets, int *perm, int n_tokens, void *stream) {
  if (!h) return fail(MOE_ERR_BAD_ARG, "null handle");
  if (n_tokens < 0 || n_tokens > h->cfg.max_tokens)
    return fail(MOE_ERR_BAD_ARG, "n_tokens %d out of range", n_tokens);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (h->unplanned.topk_i) {
    const moe_config &c = h->cfg;
    HIP_TRY(launch_dispatch(h->unplanned.topk_i, h->unplanned.pos, h->unplanned.T, c.experts,
                            gate_up_col_tiles(h), down_col_tiles(h), h->disp, s));
    h->unplanned.topk_i = nullptr;
  }
  if (offsets)
    HIP_TRY(hipMemcpyAsync(offsets, h->disp.offsets, ((size_t)h->cfg.experts + 1) * sizeof(int),
                           hipMemcpyDeviceToDevice, s));
  if (perm && n_tokens > 0)
    HIP_TRY(hipMemcpyAsync(perm, h->disp.perm, (size_t)n_tokens * kTopK * sizeof(int),
                           hipMemcpyDeviceToDevice, s));
  return MOE_OK;
}

int moe_experts(moe_handle *h, int layer, const uint16_t *x, const int *pos, const int *topk_i,
                const float *topk_v, int n_tokens, float *out, int accumulate, void *stream) {
  int rc = check_forward_args(h, layer, x, n_tokens, out);
  if (rc != MOE_OK) return rc;
  if (n_tokens == 0) return MOE_OK;
  if (!topk_i || !topk_v) return fail(MOE_ERR_BAD_ARG, "null device pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  StageTimer tm(h, s);
  HIP_TRY(tm.mark(MOE_STAGE_ROUTER));
  // ids from outside may name an expert in several slots of a token, unless the
  // caller has said otherwise (moe_set_distinct_ids)
  const int max_rows = h->distinct_ids ? n_tokens : n_tokens * kTopK;
  rc = run_experts(h, layer, x, pos, topk_i, topk_v, n_tokens, max_rows, out, accumulate, s, tm);
  if (rc == MOE_OK) tm.done();
  return rc;
}

int moe_expert_gemms(moe_handle *h, int layer, const uint16_t *x, int n_tokens, void *stream) {
  int rc = check_forward_args(h, layer, x, n_tokens, x);
  if (rc != MOE_OK) return rc;
  if (h->disp_tokens != n_tokens)
    return fail(MOE_ERR_STATE, "moe_expert_gemms(%d tokens) needs a moe_dispatch of the same batch first (last: %d)",
                n_tokens, h->disp_tokens);
  if (n_tokens == 0) return MOE_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  StageTimer tm(h, nullptr);  // stage-level calls are not timed
  tm.ev = nullptr;
  // the ids of a moe_dispatch come from outside and may name an expert in several slots of a token
  const int max_rows = h->distinct_ids ? n_tokens : n_tokens * kTopK;
  rc = run_gemms(h, layer, x, n_tokens, max_rows, DirectIds{nullptr, nullptr, 0, 0}, s, tm);
  if (rc == MOE_OK) h->gemms_done = true;
  return rc;
}

int moe_combine(moe_handle *h, const float *topk_v, const int *pos, int n_tokens, float *out,
                int accumulate, void *stream) {
  if (!h) return fail(MOE_ERR_BAD_ARG, "null handle");
  if (n_tokens < 0) return fail(MOE_ERR_BAD_ARG, "n_tokens %d is negative", n_tokens);
  if (h->disp_tokens != n_tokens)
    return fail(MOE_ERR_STATE, "moe_combine(%d tokens) needs moe_dispatch and moe_expert_gemms of the same batch first (last: %d)",
                n_tokens, h->disp_tokens);
  if (n_tokens == 0) return MOE_OK;
  if (!h->gemms_done)
    return fail(MOE_ERR_STATE, "moe_combine(%d tokens): moe_expert_gemms has not run on this dispatch", n_tokens);
  if (!topk_v || !out) return fail(MOE_ERR_BAD_ARG, "null device pointer");
  StageTimer tm(h, nullptr);
  tm.ev = nullptr;
  return run_combine(h, topk_v, pos, n_tokens, out, accumulate, nullptr, DirectIds{nullptr, nullptr, 0, 0},
                     static_cast<hipStream_t>(stream), tm);
}

int moe_forward(moe_handle *h, int layer, const uint16_t *x, const int *pos, int n_tokens,
                float *out, int accumulate, void *stream) {
  int rc = check_forward_args(h, layer, x, n_tokens, out);
  if (rc != MOE_OK) return rc;
  if (n_tokens == 0) return MOE_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const LayerWeights &lw = h->layers[layer];
  StageTimer tm(h, s);
  HIP_TRY(tm.mark(MOE_STAGE_ROUTER));
  HIP_TRY(launch_router(x, pos, lw.wr, lw.br, lw.br + h->E_pad, n_tokens, h->cfg.hidden, h->cfg.experts,
                        h->E_pad, nullptr, h->topk_i, h->topk_v, s));
  rc = run_experts(h, layer, x, pos, h->topk_i, h->topk_v, n_tokens, n_tokens, out, accumulate, s, tm);
  if (rc == MOE_OK) tm.done();
  return rc;
}

int moe_set_distinct_ids(moe_handle *h, int distinct) {
  if (!h) return fail(MOE_ERR_BAD_ARG, "null handle");
  h->distinct_ids = distinct != 0;
  return MOE_OK;
}

int moe_upload_norm(moe_handle *h, int layer, const float *rms_ffn_w) {
  const int rc0 = check_upload_args(h, layer);
  if (rc0 != MOE_OK) return rc0;
  if (!rms_ffn_w) return fail(MOE_ERR_BAD_ARG, "null weight pointer");
  const int H = h->cfg.hidden;
  LayerWeights &lw = h->layers[layer];
  int rc = MOE_OK;
  if (!lw.rms_w) rc = dev_alloc(h, &lw.rms_w, (size_t)H, false);
  if (rc == MOE_OK && !h->t_norm) rc = dev_alloc(h, &h->t_norm, (size_t)h->cfg.max_tokens * H, true);
  if (rc != MOE_OK) return rc;
  float *stage = nullptr;
  HIP_TRY(hipMalloc(reinterpret_cast<void **>(&stage), (size_t)H * sizeof(float)));
  auto body = [&]() -> int {
    HIP_TRY(hipMemcpy(stage, rms_ffn_w, (size_t)H * sizeof(float), hipMemcpyHostToDevice));
    HIP_TRY(launch_pack_bias(stage, lw.rms_w, nullptr, 1, H, H, false, nullptr));  // rounds to bf16 values
    HIP_TRY(hipDeviceSynchronize());
    return MOE_OK;
  };
  rc = body();
  (void)hipFree(stage);
  return rc;
}

int moe_block_forward(moe_handle *h, int layer, uint16_t *x, const int *pos, int n_tokens,
                      void *stream) {
  int rc = check_forward_args(h, layer, x, n_tokens, x);
  if (rc != MOE_OK) return rc;
  const LayerWeights &lw = h->layers[layer];
  if (!lw.rms_w)
    return fail(MOE_ERR_STATE, "layer %d has no norm weight (moe_upload_norm not called)", layer);
  if (n_tokens == 0) return MOE_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  StageTimer tm(h, s);
  HIP_TRY(tm.mark(MOE_STAGE_ROUTER));  // the norm is counted with the router stage
  HIP_TRY(launch_rmsnorm(x, lw.rms_w, pos, h->t_norm, n_tokens, h->cfg.hidden, s));
  HIP_TRY(launch_router(h->t_norm, pos, lw.wr, lw.br, lw.br + h->E_pad, n_tokens, h->cfg.hidden,
                        h->cfg.experts, h->E_pad, nullptr, h->topk_i, h->topk_v, s));
  rc = run_experts(h, layer, h->t_norm, pos, h->topk_i, h->topk_v, n_tokens, n_tokens, nullptr, 0, s, tm,
                   x);
  if (rc == MOE_OK) tm.done();
  return rc;
}

int moe_profile_enable(moe_handle *h, int n_calls) {
  if (!h) return fail(MOE_ERR_BAD_ARG, "null handle");
  if (n_calls < 0 || n_calls > kMaxProfileCalls)
    return fail(MOE_ERR_BAD_ARG, "n_calls %d outside [0,%d]", n_calls, kMaxProfileCalls);
  if (h->events.empty()) {
    h->events.resize((size_t)kMaxProfileCalls * (MOE_NUM_STAGES + 1), nullptr);
    for (auto &ev : h->events) {
      const hipError_t e = hipEventCreate(&ev);
      if (e != hipSuccess) {  // all events or none: later calls record into every one of them
        for (hipEvent_t made : h->events)
          if (made) (void)hipEventDestroy(made);
        h->events.clear();
        return fail(MOE_ERR_HIP, "hipEventCreate failed: %s", hipGetErrorString(e));
      }
    }
  }
  h->prof_armed = n_calls;
  h->prof_recorded = 0;
  return MOE_OK;
}

int moe_profile_read(moe_handle *h, float *ms, int *n_calls) {
  if (!h || !ms) return fail(MOE_ERR_BAD_ARG, "null argument");
  if (h->events.empty()) return fail(MOE_ERR_STATE, "profiling was never enabled");
  double sum[MOE_NUM_STAGES] = {0};
  for (int c = 0; c < h->prof_recorded; c++) {
    hipEvent_t *ev = &h->events[(size_t)c * (MOE_NUM_STAGES + 1)];
    HIP_TRY(hipEventSynchronize(ev[MOE_NUM_STAGES]));
    for (int st = 0; st < MOE_NUM_STAGES; st++) {
      float t = 0.f;
      HIP_TRY(hipEventElapsedTime(&t, ev[st], ev[st + 1]));
      sum[st] += t;
    }
  }
  for (int st = 0; st < MOE_NUM_STAGES; st++)
    ms[st] = h->prof_recorded ? (float)(sum[st] / h->prof_recorded) : 0.f;
  if (n_calls) *n_calls = h->prof_recorded;
  return MOE_OK;
}

size_t moe_weight_bytes(const moe_handle *h) { return h ? h->layer_bytes : 0; }
size_t moe_workspace_bytes(const moe_handle *h) { return h ? h->ws_bytes : 0; }

int moe_dev_alloc(void **ptr, size_t bytes) {
  if (!ptr) return fail(MOE_ERR_BAD_ARG, "null argument");
  HIP_TRY(hipMalloc(ptr, bytes ? bytes : 1));
  return MOE_OK;
}
int moe_dev_free(void *ptr) {
  HIP_TRY(hipFree(ptr));
  return MOE_OK;
}
int moe_dev_upload(void *dst_dev, const void *src_host, size_t bytes) {
  HIP_TRY(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
  return MOE_OK;
}
int moe_dev_download(void *dst_host, const void *src_dev, size_t bytes) {
  HIP_TRY(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
  return MOE_OK;
}
int moe_dev_memset(void *dst_dev, int value, size_t bytes) {
  HIP_TRY(hipMemset(dst_dev, value, bytes));
  return MOE_OK;
}
int moe_dev_sync(void) {
  HIP_TRY(hipDeviceSynchronize());
  return MOE_OK;
}
int moe_dev_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

int moe_time_forward(moe_handle *h, int layer, const uint16_t *x, const int *pos, int n_tokens,
                     float *out, int warmup, int iters, float *total_ms) {
  if (!total_ms || iters <= 0 || warmup < 0) return fail(MOE_ERR_BAD_ARG, "bad timing arguments");
  hipStream_t s = nullptr;
  HIP_TRY(hipStreamCreate(&s));
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = MOE_OK;
  auto body = [&]() -> int {
    HIP_TRY(hipEventCreate(&e0));
    HIP_TRY(hipEventCreate(&e1));
    for (int i = 0; i < warmup; i++) {
      int r = moe_forward(h, layer, x, pos, n_tokens, out, 0, s);
      if (r != MOE_OK) return r;
    }
    HIP_TRY(hipStreamSynchronize(s));
    HIP_TRY(hipEventRecord(e0, s));
    for (int i = 0; i < iters; i++) {
      int r = moe_forward(h, layer, x, pos, n_tokens, out, 0, s);
      if (r != MOE_OK) return r;
    }
    HIP_TRY(hipEventRecord(e1, s));
    HIP_TRY(hipEventSynchronize(e1));
    HIP_TRY(hipEventElapsedTime(total_ms, e0, e1));
    return MOE_OK;
  };
  rc = body();
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipStreamDestroy(s);
  return rc;
}

int moe_time_forward_each(moe_handle *h, int layer, const uint16_t *x, const int *pos, int n_tokens,
                          float *out, int iters, float *ms_each) {
  if (!ms_each || iters <= 0 || iters > 4096) return fail(MOE_ERR_BAD_ARG, "bad timing arguments");
  hipStream_t s = nullptr;
  HIP_TRY(hipStreamCreate(&s));
  std::vector<hipEvent_t> ev((size_t)iters + 1, nullptr);
  auto body = [&]() -> int {
    for (auto &e : ev) HIP_TRY(hipEventCreate(&e));
    HIP_TRY(hipEventRecord(ev[0], s));
    for (int i = 0; i < iters; i++) {
      int r = moe_forward(h, layer, x, pos, n_tokens, out, 0, s);
      if (r != MOE_OK) return r;
      HIP_TRY(hipEventRecord(ev[i + 1], s));
    }
    HIP_TRY(hipEventSynchronize(ev[iters]));
    for (int i = 0; i < iters; i++) HIP_TRY(hipEventElapsedTime(&ms_each[i], ev[i], ev[i + 1]));
    return MOE_OK;
  };
  const int rc = body();
  for (hipEvent_t e : ev)
    if (e) (void)hipEventDestroy(e);
  (void)hipStreamDestroy(s);
  return rc;
}

}  // extern "C"
