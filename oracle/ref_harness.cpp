// Builds the reference's own CPU MoE path into a shared library so that the
// oracle (moe_oracle.c) can be validated against it.  TEST INFRASTRUCTURE.
//
// The reference is compiled from the sources where they lie: REF_RUN_CPP is the
// path of its run.cpp, given on the compiler command line (see Makefile).  No
// reference source is copied here.  Only the CPU path is ever executed
// (forward(), matmul(), topk(), softmax() in run.cpp); the HIP runtime the file
// links against initialises lazily and is never touched.
#define TESTING
#include REF_RUN_CPP

#include <cstring>
#include <vector>

extern "C" {

// run.cpp:321-334
void ref_rmsnorm(float *o, float *x, float *weight, int size) { rmsnorm(o, x, weight, size); }

// run.cpp:356-369
void ref_matmul(float *xout, float *x, float *w, int n, int d) { matmul(xout, x, w, n, d); }
// run.cpp:388-421
void ref_topk(float *v, int *i, float *score, int E, int K) { topk(v, i, score, E, K); }
// run.cpp:336-354
void ref_softmax(float *x, int n) { softmax(x, n); }

// Runs forward() (run.cpp:529-758) once per row of emb on a one-layer in-memory
// Transformer whose attention block contributes exactly zero (all attention
// weights and biases are 0, so x is unchanged by run.cpp:552-657) and whose FFN
// norm scale is 1.  After each call RunState holds, for that token, the MoE
// input s->t (= rmsnorm of the embedding row, run.cpp:660), router_score,
// topk_i, topk_v (after softmax) and e_agg (run.cpp:664-745).
int ref_moe_forward(int T, int H, int IM, int E, int K, float limit,
                    const float *emb, const float *w_router, const float *b_router,
                    const float *w_mlp1, const float *b_mlp1, const float *w_mlp2,
                    const float *b_mlp2, float *t_out, float *score, int *topk_i,
                    float *topk_v, float *e_agg) {
  Transformer tr;
  std::memset(&tr, 0, sizeof(tr));
  Config &c = tr.config;
  c.vocab_size = T;
  c.hidden_dim = H;
  c.n_experts = E;
  c.experts_per_token = K;
  c.intermediate_dim = IM;
  c.n_layers = 1;
  c.head_dim = 2;
  c.n_attn_heads = 1;
  c.n_kv_heads = 1;
  c.seq_len = 1;
  c.initial_context_length = 1;
  c.rope_theta = 10000.0f;
  c.rope_scaling_factor = 1.0f; // skips the YaRN branch (run.cpp:437-470)
  c.sliding_window = 0;
  c.swiglu_limit = limit;

  const int qkv_rows = c.head_dim * (c.n_attn_heads + 2 * c.n_kv_heads);
  std::vector<float> ones(H, 1.0f), zeros_h(H, 0.0f);
  std::vector<float> w_qkv((size_t)qkv_rows * H, 0.0f), b_qkv(qkv_rows, 0.0f);
  std::vector<float> w_o((size_t)H * c.head_dim * c.n_attn_heads, 0.0f);
  std::vector<float> sinks(c.n_attn_heads, 0.0f);
  std::vector<float> unembed((size_t)T * H, 0.0f);

  TransformerWeights &w = tr.weights;
  w.token_embedding_table = const_cast<float *>(emb);
  w.rms_attn_w = ones.data();
  w.rms_ffn_w = ones.data();
  w.w_qkv = w_qkv.data();
  w.b_qkv = b_qkv.data();
  w.w_o = w_o.data();
  w.b_o = zeros_h.data();
  w.attn_sinks = sinks.data();
  w.w_router = const_cast<float *>(w_router);
  w.b_router = const_cast<float *>(b_router);
  w.w_mlp1 = const_cast<float *>(w_mlp1);
  w.b_mlp1 = const_cast<float *>(b_mlp1);
  w.w_mlp2 = const_cast<float *>(w_mlp2);
  w.b_mlp2 = const_cast<float *>(b_mlp2);
  w.rms_out_w = ones.data();
  w.out = unembed.data();

  malloc_run_state(&tr.state, &c);
  RunState &s = tr.state;
  for (int t = 0; t < T; t++) {
    forward(&tr, t, 0);
    if (t_out) std::memcpy(t_out + (size_t)t * H, s.t, sizeof(float) * H);
    if (score) std::memcpy(score + (size_t)t * E, s.router_score, sizeof(float) * E);
    if (topk_i) std::memcpy(topk_i + (size_t)t * K, s.topk_i, sizeof(int) * K);
    if (topk_v) std::memcpy(topk_v + (size_t)t * K, s.topk_v, sizeof(float) * K);
    if (e_agg) std::memcpy(e_agg + (size_t)t * H, s.e_agg, sizeof(float) * H);
  }
  free_run_state(&tr.state);
  return 0;
}

} // extern "C"
