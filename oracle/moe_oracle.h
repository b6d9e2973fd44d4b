/*
 * CPU oracle for the GPT-OSS mixture-of-experts layer.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * CPU MoE path (run.cpp) used as the checker in tests, in the smoke check and
 * as the timed CPU baseline of the benchmark.  Nothing in the product library
 * links, imports or calls it.
 *
 * Every function cites the reference lines it restates.  Citations are
 * relative to the reference checkout (pmatuan/gpt-oss).
 *
 * Pinning status (what independent evidence checks each function):
 *   oracle_matmul, oracle_topk, oracle_softmax, oracle_moe_layer (mode 0)
 *       - compared against the reference's own functions / forward() compiled
 *         from its sources (oracle/_ref), on the committed config-1 vectors and
 *         on tie fixtures; plus closed forms (one-hot x, W2 = I, E = K = 1).
 *   oracle_dispatch
 *       - the reference has no stable dispatch (its order is atomic-race
 *         order, utility.cpp:1079-1106); pinned by brute force and invariants
 *         (permutation, exclusive scan, token order inside every segment).
 *   oracle_f32_to_bf16
 *       - pinned by known-answer values of round-to-nearest-even and by an
 *         exhaustive comparison against an integer formulation.
 *   oracle_mxfp4_dequant
 *       - pinned by the 16-code x 11-exponent closed-form table.
 *   oracle_rmsnorm
 *       - the committed config-1 vectors hold the reference's own t =
 *         rmsnorm(embedding row) (unit weight); compared bit for bit; with
 *         other weights compared against the reference's rmsnorm() from
 *         oracle/_ref where that is built; closed forms (constant vector,
 *         invariance of the direction under scaling).
 *   oracle_moe_layer with ORACLE_ROUND_ACT_BF16
 *       - same control flow as mode 0; the extra rounding point is the one
 *         the reference's GPU path has (matmul.cpp:1427).  When the rounding
 *         is the identity (activations already representable) it must equal
 *         mode 0 exactly; that is tested.
 */
#ifndef MOE_ORACLE_H
#define MOE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* mode bits for oracle_moe_layer / oracle_expert_token */
#define ORACLE_ROUND_ACT_BF16 1 /* round the SwiGLU output to bf16 (matmul.cpp:1427) */
#define ORACLE_PAR_TOKENS 2     /* OpenMP over tokens instead of over output rows */

/* bf16 round-to-nearest-even, amd_hip_bfloat16.h:96-131 (ROCm) */
uint16_t oracle_f32_to_bf16(float f);
float oracle_bf16_to_f32(uint16_t h);
void oracle_round_to_bf16(float *x, size_t n); /* in place, result stays float */

/* run.cpp:356-369 -- float product, double sequential accumulate */
void oracle_matmul(float *xout, const float *x, const float *w, int n, int d);
/* run.cpp:372-421 -- descending by value; equal values keep the lower index first */
void oracle_topk(float *topk_v, int *topk_i, const float *score, int E, int K);
/* run.cpp:336-354 */
void oracle_softmax(float *x, int size);
/* run.cpp:321-334: o = weight * x / sqrt(mean(x^2) + 1e-5) */
void oracle_rmsnorm(float *o, const float *x, const float *weight, int size);

/* run.cpp:664-676 for every row with pos >= 0 (pos may be NULL = all active).
 * Inactive rows: topk_i = -1, topk_v = 0, score untouched. */
void oracle_router(const float *x, const int *pos, const float *w_router,
                   const float *b_router, int T, int H, int E, int K,
                   float *score, int *topk_i, float *topk_v);

/* Stable token->expert dispatch.  offsets[E+1] = exclusive scan of the
 * per-expert histogram over active rows; perm[offsets[e]..offsets[e+1]) lists
 * the assignments t*K+k with topk_i[t*K+k]==e in increasing token order.
 * inv[t*K+k] = position in perm, or -1 for inactive rows (inv may be NULL). */
void oracle_dispatch(const int *topk_i, const int *pos, int T, int E, int K,
                     int *offsets, int *perm, int *inv);

/* run.cpp:693-738 for one token and one expert: y = W2*swiglu(W1*t+b1)+b2.
 * scratch must hold 3*IM floats. */
void oracle_expert_token(const float *t, const float *w1, const float *b1,
                         const float *w2, const float *b2, int H, int IM,
                         float limit, int mode, float *scratch, float *y);

/* run.cpp:662-745 batched over T tokens: out[T,H] (rows with pos<0 are zero).
 * Optional outputs (may be NULL): score[T,E], topk_i[T,K], topk_v[T,K]. */
void oracle_moe_layer(const float *x, const int *pos, const float *w_router,
                      const float *b_router, const float *w_mlp1,
                      const float *b_mlp1, const float *w_mlp2,
                      const float *b_mlp2, int T, int H, int IM, int E, int K,
                      float limit, int mode, float *out, float *score,
                      int *topk_i, float *topk_v);

/* export_model_bin/gpt-oss-20b/export_model_bin.py:66-123.
 * blocks: n_blocks*16 bytes, scales: n_blocks bytes, out: n_blocks*32 floats. */
void oracle_mxfp4_dequant(const uint8_t *blocks, const uint8_t *scales,
                          size_t n_blocks, float *out);

int oracle_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
