/*
 * C-ABI of the MI355X (gfx950) GPT-OSS mixture-of-experts layer.
 *
 * Drop-in boundary for the MoE path of pmatuan/gpt-oss in getp mode.  Each
 * entry point names the reference interface it replaces (file:line relative to
 * the reference checkout).  All pointers named x / pos / out / topk_* / score
 * are DEVICE pointers unless stated otherwise; weight pointers given to the
 * upload calls are HOST pointers in the reference's host layout
 * (TransformerWeights, run.cpp:67-79, mapped at run.cpp:234-247).
 *
 * Every function returns MOE_OK (0) or a negative moe_status; the text of the
 * last failure on the calling thread is available from moe_last_error().
 * Nothing here exits the process (the reference's HIP_CHECK does,
 * common/defines.h:94-102); the host shim turns a non-zero status into that
 * behaviour.
 *
 * A handle belongs to one device and one host thread at a time.  Calls on one
 * handle are asynchronous on the given stream and never synchronise with the
 * host; all routing counts and offsets stay on the device.
 */
#ifndef MI355_MOE_ABI_H
#define MI355_MOE_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct moe_handle moe_handle;

typedef enum {
  MOE_OK = 0,
  MOE_ERR_BAD_ARG = -1,     /* null pointer, negative size, unknown layer ... */
  MOE_ERR_UNSUPPORTED = -2, /* shape outside what the kernels are built for   */
  MOE_ERR_CAPACITY = -3,    /* n_tokens > max_tokens (getp_run.cpp:532-552)   */
  MOE_ERR_HIP = -4,         /* a HIP runtime call failed                      */
  MOE_ERR_STATE = -5        /* layer not uploaded, profiling not enabled ...  */
} moe_status;

/* Model hyper-parameters of the path: Config fields hidden_dim, n_experts,
 * experts_per_token, intermediate_dim, n_layers, swiglu_limit (run.cpp:26-46).
 * max_tokens replaces MAX_BATCH_SIZE / MAX_BATCH_SIZE_120B
 * (common/defines.h:30-31). */
typedef struct {
  int hidden;        /* H,  multiple of 32 (padded to 64 inside, as the reference
                        pads its packed weights, utility/utility.cpp:558-622;
                        gpt-oss-7m has 32, export_model_bin/gpt-oss-7m/config.json:3) */
  int inter;         /* IM, multiple of 32 (likewise)          */
  int experts;       /* E,  1..256                             */
  int topk;          /* K,  must be 4 (EXPERT_PER_TOKEN)       */
  int layers;        /* number of MoE layers held by the handle */
  int max_tokens;    /* largest batch a forward call may carry */
  float swiglu_limit;
} moe_config;

/* Stage indices for moe_profile_read. */
enum {
  MOE_STAGE_ROUTER = 0,   /* logits + bias + top-4 + softmax        */
  MOE_STAGE_DISPATCH = 1, /* histogram + scan + stable permutation  */
  MOE_STAGE_GATE_UP = 2,  /* grouped GEMM 1 + clamped SwiGLU (reads the routed token rows itself) */
  MOE_STAGE_DOWN = 3,     /* grouped GEMM 2 + bias                  */
  MOE_STAGE_COMBINE = 4,  /* weighted sum back to token order       */
  MOE_NUM_STAGES = 5
};

/* Allocates weights and workspaces for cfg on the current device.
 * Replaces the allocation half of init_device_context_ep (expert.cpp:709-873)
 * and init_device_context (getp_run.cpp:19-185). */
int moe_create(const moe_config *cfg, moe_handle **out);

/* Frees everything the handle owns.  Replaces cleanup_device_context_ep
 * (expert.cpp:1234-1364). */
int moe_destroy(moe_handle *h);

/* Converts one layer's weights to bf16 (round to nearest even) and stores them
 * in the device layout of the kernels.  Arguments are the reference's host
 * pointers for that layer: w_router [E,H], b_router [E], w_mlp1 [E,2*IM,H]
 * (rows alternate gate/up), b_mlp1 [E,2*IM], w_mlp2 [E,H,IM], b_mlp2 [E,H],
 * all fp32 row-major (run.cpp:234-247).  Replaces the upload half of
 * init_device_context_ep (expert.cpp:874-1009), getp_run.cpp:186-293 and
 * pack_fp32_to_bf16_matmul (utility/utility.cpp:558-622).  Synchronous. */
int moe_upload_layer(moe_handle *h, int layer, const float *w_router,
                     const float *b_router, const float *w_mlp1,
                     const float *b_mlp1, const float *w_mlp2,
                     const float *b_mlp2);

/* As moe_upload_layer, with the expert matrices in MXFP4 as the GPT-OSS
 * checkpoints hold them: for a matrix [rows, cols] (cols a multiple of 32)
 * blocks is u8 [E, rows, cols/32, 16] and scales u8 [E, rows, cols/32]; byte b
 * of a block holds element 2b in its low and element 2b+1 in its high nibble, a
 * nibble indexes {0, .5, 1, 1.5, 2, 3, 4, 6, -0, -.5, -1, -1.5, -2, -3, -4, -6}
 * and the scale byte s multiplies by 2^(s-127) (s in 1..254).  Takes the place
 * of dequantize_fp4 in the exporter
 * (export_model_bin/gpt-oss-20b/export_model_bin.py:66-123) followed by the fp32
 * upload.  The matrices stay MXFP4 in device memory (a quarter of the bytes of
 * bf16); the GEMMs turn them into bf16 matrix-core operands in registers, which
 * is exact, so the layer's results are those of an upload of the decoded
 * matrices, bit for bit.
 * Router weights and all biases stay fp32 arguments.  Synchronous. */
int moe_upload_layer_mxfp4(moe_handle *h, int layer, const float *w_router,
                           const float *b_router,
                           const uint8_t *w_mlp1_blocks,
                           const uint8_t *w_mlp1_scales, const float *b_mlp1,
                           const uint8_t *w_mlp2_blocks,
                           const uint8_t *w_mlp2_scales, const float *b_mlp2);

/* The whole layer for one batch: out[t,:] (+)= sum_k w[t,k] * expert_k(x[t,:]).
 *   x    bf16 [n_tokens, H] row-major (the reference's d_t)
 *   pos  int  [n_tokens] or NULL; pos[t] < 0 marks an inactive row, which takes
 *        part in nothing (utility.cpp:281-282, :1071; matmul.cpp:955)
 *   out  f32  [n_tokens, H] (the reference's d_e_agg).  accumulate != 0: the
 *        result is added to out, as the reference does after zeroing it
 *        (getp_run.cpp:719-720, utility.cpp:719-724); accumulate == 0: out is
 *        overwritten and inactive rows are set to zero.
 * Replaces getp_run.cpp:697-845 (router, top-k, local MoE path) and, with one
 * GPU, gpu_forward_device_batch_ep (expert.cpp:1366-1607). */
int moe_forward(moe_handle *h, int layer, const uint16_t *x, const int *pos,
                int n_tokens, float *out, int accumulate, void *stream);

/* The weight of the RMS norm in front of the layer (rms_ffn_w + layer*H,
 * run.cpp:51, used at run.cpp:660; device copy d_rms_ffn_w, getp_run.cpp:691),
 * fp32 [H]; kept as bf16 values like the other weights.  Needed by
 * moe_block_forward only.  Synchronous. */
int moe_upload_norm(moe_handle *h, int layer, const float *rms_ffn_w);

/* The FFN block in place on the residual stream x (bf16 [n_tokens, H], the
 * reference's d_x):  t = rmsnorm(x) * rms_ffn_w;  x = bf16(x + layer(t)).
 * Replaces rmsnorm_batch_kernel (utility/utility.cpp:194-271, launched at
 * getp_run.cpp:688-695), the layer itself as moe_forward, and
 * residual_add_batch_kernel (utility/utility.cpp:158-173, launched at
 * getp_run.cpp:846-852); on the CPU path run.cpp:660-750.  The normalised rows
 * and the fp32 sum never leave the library's workspace.  Rows with pos < 0 are
 * left as they are.  Asynchronous on `stream`. */
int moe_block_forward(moe_handle *h, int layer, uint16_t *x, const int *pos,
                      int n_tokens, void *stream);

/* The router stage alone.  Writes topk_i int [n_tokens,K] (descending score,
 * ties to the lower expert id; -1 on inactive rows), topk_v f32 [n_tokens,K]
 * (softmax over the K selected logits) and, if score != NULL, the logits f32
 * [n_tokens,E].  Replaces matmul_router_kernel (matmul/matmul.cpp:945-1019)
 * and fused_topk_softmax_batch_kernel (utility/utility.cpp:273-365), i.e. the
 * producers of d_router_score, d_topk_i, d_topk_v (getp_run.cpp:697-716).
 * Accuracy: topk_i is exactly what the CPU path's arithmetic selects (float
 * products summed in a double, run.cpp:363-369).  That arithmetic is carried
 * out only for the logits that decide a selection; all other entries of score,
 * and topk_v of tokens whose selection was clear from the first pass, come from
 * a bf16 matrix-core pass with fp64 hand-over and lie within 2e-6 + 2^-22
 * relative of the exact values. */
int moe_router(moe_handle *h, int layer, const uint16_t *x, const int *pos,
               int n_tokens, float *score, int *topk_i, float *topk_v,
               void *stream);

/* Stage 2 alone, from caller-supplied routing.  Builds, inside the handle,
 * offsets int [E+1] (exclusive scan of the per-expert histogram over active
 * rows) and perm int [offsets[E]]: segment e lists the assignments t*K+k with
 * topk_i[t,k] == e in increasing token order.  Replaces
 * count_expert_assignments_kernel, exclusive_scan_small_kernel and
 * build_expert_assignments_kernel (utility/utility.cpp:1058-1106, :758-777). */
int moe_dispatch(moe_handle *h, const int *topk_i, const int *pos, int n_tokens,
                 void *stream);

/* Copies the result of the last dispatch to device buffers of the caller:
 * offsets int [E+1], perm int [n_tokens*K] (entries past offsets[E] are -1).
 * Either may be NULL.  The last dispatch is that of moe_dispatch or of the last
 * moe_forward / moe_experts / moe_block_forward.  Those three need no dispatch
 * pass for a batch of at most 64 tokens; after such a call this function runs
 * it, on `stream`, from the ids and pos of that call, which must still be
 * valid (moe_forward and moe_block_forward keep their ids in the handle). */
int moe_get_dispatch(moe_handle *h, int *offsets, int *perm, int n_tokens,
                     void *stream);

/* Everything after the router (dispatch, both GEMMs, combine) from
 * caller-supplied routing: the body of gpu_forward_device_batch_ep
 * (expert.cpp:1366), which reads d_t, d_topk_i, d_topk_v, d_pos and adds into
 * d_e_agg. */
int moe_experts(moe_handle *h, int layer, const uint16_t *x, const int *pos,
                const int *topk_i, const float *topk_v, int n_tokens,
                float *out, int accumulate, void *stream);

/* Promise about caller-supplied ids (moe_experts, moe_dispatch +
 * moe_expert_gemms): distinct != 0 says that the K ids of a token name K
 * different experts, which holds for any top-k selection, the reference's
 * included (run.cpp:388-421, utility/utility.cpp:273-365).  No expert then gets
 * more rows than the batch has tokens, and batches of up to 64 tokens run the
 * small-batch kernels (no dispatch pass, several workgroups per CU) as they do
 * under moe_forward.  Without the promise (the default) an expert may be named
 * in all K slots of every token and only batches of up to 16 tokens take that
 * path.  Ids that break the promise do not fault: rows beyond an expert's 64
 * are dropped.  Has no counterpart in the reference. */
int moe_set_distinct_ids(moe_handle *h, int distinct);

/* moe_dispatch for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  No handle is needed and no allocating
 * routine is called: the kernels' working buffers live in a device array that
 * is part of the library image (about 330 KB per GPU, held until the process
 * ends).  Inputs as moe_dispatch; the results go to the caller's device
 * buffers offsets int [n_experts+1] and perm int [n_tokens*K] (entries past
 * offsets[n_experts] are -1), bit-identical to moe_dispatch + moe_get_dispatch.
 * Limits: n_tokens <= MOE_DISPATCH_STATIC_MAX_TOKENS, n_experts <=
 * MOE_DISPATCH_STATIC_MAX_EXPERTS, otherwise MOE_ERR_CAPACITY.  All calls on
 * one GPU share the array: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered.  The first call on a device
 * looks up the array's address (hipGetSymbolAddress); make it outside a graph
 * capture. */
#define MOE_DISPATCH_STATIC_MAX_TOKENS 8192
#define MOE_DISPATCH_STATIC_MAX_EXPERTS 256
int moe_dispatch_static(const int *topk_i, const int *pos, int n_tokens,
                        int n_experts, int *offsets, int *perm, void *stream);

/* MOE_STAGE_GATE_UP and MOE_STAGE_DOWN alone, on the plan of the last
 * moe_dispatch of the same batch: the gate_up grouped GEMM with the clamped
 * SwiGLU, which reads the routed token rows of x itself through the plan's row
 * map (there is no gathered copy), then the down grouped GEMM; leaves one fp32
 * row per assignment inside the handle.  Replaces the mlp1 / mlp2 launches of
 * the local path (getp_run.cpp:788-829; kernels matmul/matmul.cpp:1023-1914). */
int moe_expert_gemms(moe_handle *h, int layer, const uint16_t *x, int n_tokens,
                     void *stream);

/* MOE_STAGE_COMBINE alone, after moe_dispatch and moe_expert_gemms of the same
 * batch (MOE_ERR_STATE if either has not run since the last dispatch):
 * out[t,:] (+)= sum_k topk_v[t,k] * (row of assignment t*K+k), slots added in
 * order 0..K-1, rows with pos < 0 skipped (accumulate) or zeroed.  Replaces
 * reduce_mlp2_slots_kernel (utility/utility.cpp:701-726, launched at
 * getp_run.cpp:831-843); the routing weight is applied here, in fp32, rather
 * than in the down GEMM's epilogue (matmul/matmul.cpp:1868-1870). */
int moe_combine(moe_handle *h, const float *topk_v, const int *pos, int n_tokens,
                float *out, int accumulate, void *stream);

/* Per-stage timing with HIP events on the stream of the forward calls.
 * moe_profile_enable(h, n) arms timing for the next n forward calls (n <= 256);
 * moe_profile_read synchronises on the recorded events and returns the mean
 * duration of every stage in milliseconds (ms[MOE_NUM_STAGES]) and the number
 * of calls measured.  Replaces PROFILE_GPU_SCOPE (profiler/profiler.h:10-18). */
int moe_profile_enable(moe_handle *h, int n_calls);
int moe_profile_read(moe_handle *h, float *ms, int *n_calls);

/* Sizes the kernels work with, for reports: number of row tiles the last
 * dispatch produced is data dependent and stays on the device; these are the
 * static figures. */
size_t moe_weight_bytes(const moe_handle *h);    /* device bytes of one layer */
size_t moe_workspace_bytes(const moe_handle *h); /* device bytes of workspaces */

const char *moe_last_error(void);
const char *moe_version(void);

/* Device-memory helpers so that a host without a HIP toolchain (the ctypes test
 * harness) can stage buffers.  Thin wrappers over hipMalloc / hipFree /
 * hipMemcpy / hipMemset / hipDeviceSynchronize; not part of the reference. */
int moe_dev_alloc(void **ptr, size_t bytes);
int moe_dev_free(void *ptr);
int moe_dev_upload(void *dst_dev, const void *src_host, size_t bytes);
int moe_dev_download(void *dst_host, const void *src_dev, size_t bytes);
int moe_dev_memset(void *dst_dev, int value, size_t bytes);
int moe_dev_sync(void);
int moe_dev_count(void);

/* Wall-clock timing of back-to-back forward calls with HIP events on one
 * stream: runs warmup untimed calls, then iters timed calls, and returns the
 * total milliseconds of the timed calls.  Used by the benchmark. */
int moe_time_forward(moe_handle *h, int layer, const uint16_t *x, const int *pos,
                     int n_tokens, float *out, int warmup, int iters,
                     float *total_ms);

/* The same with one HIP event after every call: ms_each[i] is the duration of
 * call i (iters <= 4096), for the median the benchmark reports. */
int moe_time_forward_each(moe_handle *h, int layer, const uint16_t *x,
                          const int *pos, int n_tokens, float *out, int iters,
                          float *ms_each);

/* Measured denominators for the rooflines the benchmark reports (the published
 * peaks are 2.5 PFLOP/s dense bf16 and 8 TB/s).  They take the place of the
 * reference's tuning harness (getp-csrc/matmul/tune.cpp:1347-1595, results in
 * matmul/log.txt), which times its GEMM kernels against each other only.  Not
 * used by the layer; both allocate and free their own buffers and synchronise.
 *
 * moe_yardstick_mfma: n_workgroups workgroups of 4 waves (one per SIMD, one
 * workgroup per CU up to the CU count) run v_mfma_f32_32x32x16_bf16 on 16
 * independent accumulators each from registers alone, iters x 16 per wave.
 * data 1: pseudo-random operands of unit scale; data 2: unit scale against a
 * scale of 0.02, as activations meet weights in the layer; data 0: zeros (the
 * clock the matrix cores sustain depends on the bits that toggle).  Returns
 * TFLOP/s over the launch and the mean shader clock in GHz during the loop.
 *
 * moe_yardstick_hbm: a copy kernel and a read-only kernel over `bytes` of
 * device memory (choose it well above the 256 MB memory-side cache), iters
 * launches each; copy_gbs counts bytes read plus bytes written. */
int moe_yardstick_mfma(int n_workgroups, int iters, int data, double *tflops,
                       double *shader_ghz);
int moe_yardstick_hbm(size_t bytes, int iters, double *copy_gbs, double *read_gbs);

#ifdef __cplusplus
}
#endif
#endif /* MI355_MOE_ABI_H */
