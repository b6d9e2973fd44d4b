/*
 * CPU oracle for the GPT-OSS mixture-of-experts layer -- TEST INFRASTRUCTURE.
 * See moe_oracle.h for scope, citations and pinning status.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -fPIC -shared (no -march=native:
 * the library is built on one machine and run on another).
 */
#include "moe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- bf16 (amd_hip_bfloat16.h:96-131: round to nearest, ties to even) ---- */

uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if (~u & 0x7f800000u) {
    u += 0x7fffu + ((u >> 16) & 1u);
  } else if (u & 0xffffu) {
    u |= 0x10000u; /* keep a NaN a NaN */
  }
  return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

void oracle_round_to_bf16(float *x, size_t n) {
  for (size_t i = 0; i < n; i++) x[i] = oracle_bf16_to_f32(oracle_f32_to_bf16(x[i]));
}

/* ---- run.cpp:356-369 ---- */
void oracle_matmul(float *xout, const float *x, const float *w, int n, int d) {
  int i;
#pragma omp parallel for private(i)
  for (i = 0; i < d; i++) {
    double val = 0.0;
    const float *wi = w + (size_t)i * (size_t)n;
    for (int j = 0; j < n; j++) {
      float p = wi[j] * x[j]; /* the product is rounded to float first */
      val += p;
    }
    xout[i] = (float)val;
  }
}

/* ---- run.cpp:372-421 ----
 * The reference sorts (value,index) pairs with qsort and a comparator that
 * returns 0 for equal values; under glibc's merge sort that leaves equal
 * values in index order.  Here the rule is explicit: value descending, then
 * index ascending. */
void oracle_topk(float *topk_v, int *topk_i, const float *score, int E, int K) {
  if (E <= 0 || K <= 0 || K > E) return; /* run.cpp:390-396 */
  for (int k = 0; k < K; k++) {
    int best = -1;
    for (int e = 0; e < E; e++) {
      int taken = 0;
      for (int q = 0; q < k; q++) taken |= (topk_i[q] == e);
      if (taken) continue;
      if (best < 0 || score[e] > score[best]) best = e; /* strict: lower index wins ties */
    }
    topk_i[k] = best;
    topk_v[k] = score[best];
  }
}

/* ---- run.cpp:321-334 ---- */
void oracle_rmsnorm(float *o, const float *x, const float *weight, int size) {
  double ss = 0.0f;
  for (int j = 0; j < size; j++) ss += x[j] * x[j]; /* float product, double sum */
  ss /= size;
  ss += 1e-5f;
  ss = 1.0f / sqrtf(ss); /* the argument is narrowed to float */
  for (int j = 0; j < size; j++) o[j] = weight[j] * (ss * x[j]);
}

/* ---- run.cpp:336-354 ---- */
void oracle_softmax(float *x, int size) {
  double max_val = x[0];
  for (int i = 1; i < size; i++)
    if (x[i] > max_val) max_val = x[i];
  double sum = 0.0;
  for (int i = 0; i < size; i++) {
    x[i] = expf((float)((double)x[i] - max_val));
    sum += x[i];
  }
  for (int i = 0; i < size; i++) x[i] = (float)((double)x[i] / sum);
}

/* ---- run.cpp:664-676 per active row ---- */
void oracle_router(const float *x, const int *pos, const float *w_router,
                   const float *b_router, int T, int H, int E, int K,
                   float *score, int *topk_i, float *topk_v) {
  int t;
#pragma omp parallel for private(t)
  for (t = 0; t < T; t++) {
    int *ti = topk_i + (size_t)t * K;
    float *tv = topk_v + (size_t)t * K;
    if (pos && pos[t] < 0) {
      for (int k = 0; k < K; k++) { ti[k] = -1; tv[k] = 0.0f; }
      continue;
    }
    float *sc = score + (size_t)t * E;
    oracle_matmul(sc, x + (size_t)t * H, w_router, H, E);
    for (int e = 0; e < E; e++) sc[e] += b_router[e];
    oracle_topk(tv, ti, sc, E, K);
    oracle_softmax(tv, K);
  }
}

/* ---- stable dispatch (counting sort by expert, token order kept) ---- */
void oracle_dispatch(const int *topk_i, const int *pos, int T, int E, int K,
                     int *offsets, int *perm, int *inv) {
  int *cursor = (int *)calloc((size_t)E + 1, sizeof(int));
  for (int e = 0; e <= E; e++) offsets[e] = 0;
  for (int t = 0; t < T; t++) {
    if (pos && pos[t] < 0) continue;
    for (int k = 0; k < K; k++) offsets[topk_i[(size_t)t * K + k] + 1]++;
  }
  for (int e = 0; e < E; e++) offsets[e + 1] += offsets[e];
  for (int e = 0; e < E; e++) cursor[e] = offsets[e];
  for (int t = 0; t < T; t++) {
    for (int k = 0; k < K; k++) {
      size_t a = (size_t)t * K + k;
      if (pos && pos[t] < 0) {
        if (inv) inv[a] = -1;
        continue;
      }
      int p = cursor[topk_i[a]]++;
      perm[p] = (int)a;
      if (inv) inv[a] = p;
    }
  }
  free(cursor);
}

/* ---- run.cpp:693-738 ---- */
void oracle_expert_token(const float *t, const float *w1, const float *b1,
                         const float *w2, const float *b2, int H, int IM,
                         float limit, int mode, float *scratch, float *y) {
  float *mlp1_out = scratch;      /* [2*IM] */
  float *gate_up = scratch + 2 * (size_t)IM; /* [IM] */
  oracle_matmul(mlp1_out, t, w1, H, 2 * IM);
  for (int i = 0; i < 2 * IM; i++) mlp1_out[i] += b1[i];
  const float alpha = 1.702f;
  for (int i = 0; i < IM; i++) {
    float val = mlp1_out[2 * i];        /* gate, run.cpp:703-706 */
    float up_val = mlp1_out[2 * i + 1]; /* up */
    if (val > limit) val = limit;       /* run.cpp:714-719 */
    if (up_val > limit) up_val = limit;
    if (up_val < -limit) up_val = -limit;
    val *= (1.0f / (1.0f + expf(-alpha * val)));
    val *= (up_val + 1.0f);
    if (mode & ORACLE_ROUND_ACT_BF16) val = oracle_bf16_to_f32(oracle_f32_to_bf16(val));
    gate_up[i] = val;
  }
  oracle_matmul(y, gate_up, w2, IM, H);
  for (int i = 0; i < H; i++) y[i] += b2[i];
}

/* ---- run.cpp:662-745 ---- */
void oracle_moe_layer(const float *x, const int *pos, const float *w_router,
                      const float *b_router, const float *w_mlp1,
                      const float *b_mlp1, const float *w_mlp2,
                      const float *b_mlp2, int T, int H, int IM, int E, int K,
                      float limit, int mode, float *out, float *score,
                      int *topk_i, float *topk_v) {
  int t;
  const int par = (mode & ORACLE_PAR_TOKENS) != 0;
#pragma omp parallel for private(t) schedule(dynamic, 1) if (par)
  for (t = 0; t < T; t++) {
    float *e_agg = out + (size_t)t * H;
    memset(e_agg, 0, (size_t)H * sizeof(float));
    float *sc = (float *)malloc(((size_t)E + K) * sizeof(float) + (size_t)K * sizeof(int));
    float *tv = sc + E;
    int *ti = (int *)(tv + K);
    if (pos && pos[t] < 0) {
      for (int k = 0; k < K; k++) { ti[k] = -1; tv[k] = 0.0f; }
    } else {
      const float *tx = x + (size_t)t * H;
      float *scratch = (float *)malloc((3 * (size_t)IM + H) * sizeof(float));
      float *tb2 = scratch + 3 * (size_t)IM;
      oracle_matmul(sc, tx, w_router, H, E);
      for (int e = 0; e < E; e++) sc[e] += b_router[e];
      oracle_topk(tv, ti, sc, E, K);
      oracle_softmax(tv, K);
      for (int e = 0; e < E; e++) { /* ascending expert id, run.cpp:680 */
        float expert_w = 0;
        int in_topk = 0;
        for (int idx = 0; idx < K; idx++) {
          if (ti[idx] == e) { in_topk = 1; expert_w = tv[idx]; break; }
        }
        if (!in_topk) continue;
        oracle_expert_token(tx, w_mlp1 + (size_t)e * 2 * IM * H,
                            b_mlp1 + (size_t)e * 2 * IM,
                            w_mlp2 + (size_t)e * H * IM, b_mlp2 + (size_t)e * H,
                            H, IM, limit, mode, scratch, tb2);
        for (int i = 0; i < H; i++) e_agg[i] += tb2[i] * expert_w; /* run.cpp:741-743 */
      }
      if (score) memcpy(score + (size_t)t * E, sc, (size_t)E * sizeof(float));
      free(scratch);
    }
    if (topk_i) memcpy(topk_i + (size_t)t * K, ti, (size_t)K * sizeof(int));
    if (topk_v) memcpy(topk_v + (size_t)t * K, tv, (size_t)K * sizeof(float));
    free(sc);
  }
}

/* ---- export_model_bin.py:66-123 ---- */
void oracle_mxfp4_dequant(const uint8_t *blocks, const uint8_t *scales,
                          size_t n_blocks, float *out) {
  static const float lut[16] = {+0.0f, +0.5f, +1.0f, +1.5f, +2.0f, +3.0f, +4.0f, +6.0f,
                                -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
  for (size_t g = 0; g < n_blocks; g++) {
    int exp = (int)scales[g] - 127;
    for (int b = 0; b < 16; b++) {
      uint8_t byte = blocks[g * 16 + b];
      out[g * 32 + 2 * b] = ldexpf(lut[byte & 0x0f], exp);   /* low nibble -> even */
      out[g * 32 + 2 * b + 1] = ldexpf(lut[byte >> 4], exp); /* high nibble -> odd */
    }
  }
}
