// Host-side shim (C++17): the reference's MoE entry points on top of the C-ABI
// of libmi355_moe (include/moe_abi.h).  It is meant to be #included from the
// reference's getp-csrc/getp_run.cpp (after common/defines.h, which provides
// DeviceContext, Transformer, model_config and HIP_CHECK) in place of the MoE
// kernels it launches: one call in init_device_context, one in the layer loop
// of gpu_forward_device_batch, one in cleanup_device_context.
//
// Mirrored interfaces (reference file:line):
//   mi355_moe_init      <- expert upload of init_device_context (getp_run.cpp:186-293)
//                          and init_device_context_ep (expert.cpp:874-1009)
//   mi355_moe_forward   <- gpu_forward_device_batch_ep(ctx, swiglu_limit, H, IM, E, L, K,
//                          batch_size, layer) (expert.cpp:1366): same parameter
//                          list, same buffers read (d_t, d_pos, d_topk_i, d_topk_v)
//                          and written (d_e_agg, by +=), same stream (null stream,
//                          getp_run.cpp:798), no host synchronisation
//   mi355_moe_forward_fused <- the same plus the router and top-k launches it
//                          makes redundant (getp_run.cpp:697-716)
//   mi355_moe_block     <- the whole FFN block of a layer: rmsnorm_batch_kernel, router,
//                          top-k, local MoE path and residual_add_batch_kernel
//                          (getp_run.cpp:686-852), in place on d_x
//   mi355_moe_cleanup   <- cleanup_device_context_ep (expert.cpp:1234-1364)
// Error behaviour follows HIP_CHECK (common/defines.h:94-102): print and exit.
#pragma once

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "moe_abi.h"

#define MI355_MOE_CHECK(call)                                                          \
  do {                                                                                 \
    int rc_ = (call);                                                                  \
    if (rc_ != MOE_OK) {                                                               \
      fprintf(stderr, "mi355 moe error at %s:%d - %s (status %d)\n", __FILE__, __LINE__, \
              moe_last_error(), rc_);                                                  \
      exit(EXIT_FAILURE);                                                              \
    }                                                                                  \
  } while (0)

// One handle per device, indexed by DeviceContext::device_id.
static std::vector<moe_handle *> g_mi355_moe;

static inline moe_handle *mi355_moe_of(const DeviceContext &ctx) {
  if (ctx.device_id < 0 || (size_t)ctx.device_id >= g_mi355_moe.size() ||
      !g_mi355_moe[ctx.device_id]) {
    fprintf(stderr, "mi355 moe: device %d was not initialised\n", ctx.device_id);
    exit(EXIT_FAILURE);
  }
  return g_mi355_moe[ctx.device_id];
}

// Call once per device after hipSetDevice(device_id), e.g. at the end of
// init_device_context.  max_batch is the largest batch_size the runner will
// pass (MAX_BATCH_SIZE / MAX_BATCH_SIZE_120B in the reference, defines.h:30-31).
static void mi355_moe_init(DeviceContext &ctx, int device_id, Transformer *transformer,
                           int max_batch) {
  const Config *p = &transformer->config;
  const TransformerWeights *w = &transformer->weights;
  moe_config cfg;
  cfg.hidden = p->hidden_dim;
  cfg.inter = p->intermediate_dim;
  cfg.experts = p->n_experts;
  cfg.topk = p->experts_per_token;
  cfg.layers = p->n_layers;
  cfg.max_tokens = max_batch;
  cfg.swiglu_limit = p->swiglu_limit;
  if ((size_t)device_id >= g_mi355_moe.size()) g_mi355_moe.resize(device_id + 1, nullptr);
  MI355_MOE_CHECK(moe_create(&cfg, &g_mi355_moe[device_id]));
  // d_topk_i comes from the runner's top-k (utility/utility.cpp:273-365): K different experts per token
  MI355_MOE_CHECK(moe_set_distinct_ids(g_mi355_moe[device_id], 1));
  const size_t E = p->n_experts, H = p->hidden_dim, IM = p->intermediate_dim;
  for (int l = 0; l < p->n_layers; l++) {
    // layer offsets of run.cpp:664-665, :687-690, :729-733
    MI355_MOE_CHECK(moe_upload_layer(
        g_mi355_moe[device_id], l, w->w_router + (size_t)l * H * E, w->b_router + (size_t)l * E,
        w->w_mlp1 + (size_t)l * E * 2 * IM * H, w->b_mlp1 + (size_t)l * E * 2 * IM,
        w->w_mlp2 + (size_t)l * E * H * IM, w->b_mlp2 + (size_t)l * E * H));
    // the reference's device copy is d_rms_ffn_w (getp_run.cpp:161-163)
    MI355_MOE_CHECK(moe_upload_norm(g_mi355_moe[device_id], l, w->rms_ffn_w + (size_t)l * H));
  }
  (void)ctx;
}

// Drop-in for gpu_forward_device_batch_ep (expert.cpp:1366) and for the local
// path of getp_run.cpp:725-845: the caller has run the router and top-k and
// zeroed d_e_agg (getp_run.cpp:697-720).
static void mi355_moe_forward(DeviceContext &ctx, const float swiglu_limit, const int H,
                              const int IM, const int E, const int L, const int K, int batch_size,
                              int layer) {
  (void)swiglu_limit; (void)H; (void)IM; (void)E; (void)L; (void)K;  // fixed at mi355_moe_init
  MI355_MOE_CHECK(moe_experts(mi355_moe_of(ctx), layer,
                              reinterpret_cast<const uint16_t *>(ctx.gpu_activations.d_t),
                              ctx.gpu_activations.d_pos, ctx.gpu_activations.d_topk_i,
                              ctx.gpu_activations.d_topk_v, batch_size,
                              ctx.gpu_activations.d_e_agg, /*accumulate=*/1, /*stream=*/nullptr));
}

// The same with the router fused in: replaces getp_run.cpp:697-845 (router GEMV,
// top-k + softmax, memset of d_e_agg, local MoE path).  d_e_agg is overwritten.
static void mi355_moe_forward_fused(DeviceContext &ctx, int batch_size, int layer) {
  MI355_MOE_CHECK(moe_forward(mi355_moe_of(ctx), layer,
                              reinterpret_cast<const uint16_t *>(ctx.gpu_activations.d_t),
                              ctx.gpu_activations.d_pos, batch_size, ctx.gpu_activations.d_e_agg,
                              /*accumulate=*/0, /*stream=*/nullptr));
}

// The FFN block of one layer in place on the residual stream d_x: replaces
// getp_run.cpp:686-852 (rmsnorm_batch_kernel into d_t, router, top-k, memset of
// d_e_agg, local MoE path, residual_add_batch_kernel).  d_t and d_e_agg are not
// touched.
static void mi355_moe_block(DeviceContext &ctx, int batch_size, int layer) {
  MI355_MOE_CHECK(moe_block_forward(mi355_moe_of(ctx), layer,
                                    reinterpret_cast<uint16_t *>(ctx.gpu_activations.d_x),
                                    ctx.gpu_activations.d_pos, batch_size, /*stream=*/nullptr));
}

static void mi355_moe_cleanup(DeviceContext &ctx) {
  if (ctx.device_id >= 0 && (size_t)ctx.device_id < g_mi355_moe.size() &&
      g_mi355_moe[ctx.device_id]) {
    MI355_MOE_CHECK(moe_destroy(g_mi355_moe[ctx.device_id]));
    g_mi355_moe[ctx.device_id] = nullptr;
  }
}

#ifdef MI355_MOE_REPLACE_EP
// The reference's own entry points (getp-csrc/expert.cpp) under their own names,
// for a runner that takes its `use_expert_parallelism` branch (getp_run.cpp:408,
// :434, :723) and whose expert.cpp no longer carries the MoE code -- see
// shim/expert.cpp, which takes the place of that file.  One GPU: every expert is
// local, so there is no exchange between devices.

// init_device_context_ep (expert.cpp:709): everything that is not the MoE layer
// (activations, attention and embedding weights, KV cache, streams) is set up by
// the reference's own init_device_context (getp_run.cpp:19), defined further
// down in the same translation unit; the expert weights go to libmi355_moe.
static void init_device_context(DeviceContext &ctx, int device_id, Transformer *transformer);
static void init_device_context_ep(DeviceContext &ctx, int device_id, Transformer *transformer) {
  init_device_context(ctx, device_id, transformer);
  mi355_moe_init(ctx, device_id, transformer, MAX_BATCH_SIZE);
}

// warm_up_ep (expert.cpp:1176): the reference builds its owner maps and enables
// peer access here; with all experts on the one device only the per-device
// initialisation is left (the same loop as expert.cpp:1216-1218).
static void warm_up_ep(Transformer *transformer) {
  for (int i = 0; i < g_num_devices; ++i) init_device_context_ep(g_devices[i], i, transformer);
}

// gpu_forward_device_batch_ep (expert.cpp:1366): same parameter list; the caller
// has run the router and the top-k and zeroed d_e_agg (getp_run.cpp:697-720).
static void gpu_forward_device_batch_ep(DeviceContext &ctx, const float swiglu_limit, const int H,
                                        const int IM, const int E, const int L, const int K,
                                        int batch_size, int layer) {
  mi355_moe_forward(ctx, swiglu_limit, H, IM, E, L, K, batch_size, layer);
}

// cleanup_device_context_ep (expert.cpp:1234): called by the reference's
// cleanup_device_context after it has freed its own buffers (getp_run.cpp:408-410).
static void cleanup_device_context_ep(DeviceContext &ctx) { mi355_moe_cleanup(ctx); }
#endif
