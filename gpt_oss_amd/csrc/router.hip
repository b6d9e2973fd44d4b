// Router: logits = x * Wr^T + br, top-4 with ties to the lower expert id,
// softmax over the four selected logits.  Replaces matmul_router_kernel
// (matmul/matmul.cpp:945-1019) and fused_topk_softmax_batch_kernel
// (utility/utility.cpp:273-365).  The expert ids must be those of the
// reference's CPU path (run.cpp:356-369 matmul: float products accumulated in a
// double, rounded to float once; :669-671 bias added in float; :388-421 top-k;
// :336-354 softmax), bit for bit.
//
// Two passes in one kernel:
//   1. All logits on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16).  The
//      products are exact; the fp32 accumulation inside the matrix core is not,
//      so a wave hands its fp32 sums over to fp64 accumulators every FLUSH
//      MFMAs (every one while the experts are few and the hand-over is cheap).
//      That bounds the error of a logit by gamma * sum_k |x_k w_ek|
//      <= gamma * |x| * |w_e| (Cauchy-Schwarz; |x|^2 comes out of one more
//      MFMA per chunk, x times its own transpose, and max_e |w_e| is computed
//      at upload).
//   2. A token whose five best logits are further apart than twice that bound
//      is decided: ids, order and (to about 1e-7) weights are those of the
//      exact arithmetic.  For any other token the experts that can still reach
//      the top four -- those within the bound of the fourth best -- get their
//      logit recomputed exactly: float products (exact for bf16 factors)
//      summed in fp64, rounded to float once, bias added in float, which is the
//      arithmetic of run.cpp:363-369 up to the order of the fp64 additions.
//      An expert outside that set is below four experts by more than the two
//      error bounds, so it cannot be among the exact top four; inside the set
//      all values are exact, so the selection (value descending, index
//      ascending) is the reference's.
// At the benchmark shapes a few per cent of the tokens take the second pass,
// with four to six experts each, instead of every token paying fp64 for every
// expert.
#include "moe_internal.h"

namespace moe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Error of one fp32 chain of `flush` MFMAs (of 32 k each) started from zero,
// relative to the sum of the magnitudes of its 32 * flush products: every one
// of its 33 * flush additions is taken to lose at most 2^-23 of the running
// magnitude (covers truncation as well as rounding), and the result is doubled.
__host__ __device__ constexpr float router_gamma(int flush) { return 2.0f * 33.0f * flush * 1.1920929e-7f; }
constexpr int kNone = 0x7fffffff;

// Top-NSEL of a token's logits held by LPT neighbouring lanes (lane q of them
// owns experts q*PER .. q*PER+PER-1), by the rule of the reference's CPU top-k under a stable
// sort: value descending, index ascending; a candidate replaces the incumbent
// (the one with the lower index) only if it compares strictly greater, so a
// NaN neither wins nor loses a comparison and a row of NaNs selects 0, 1, 2, 3.
// Experts >= E are never selected.  All LPT lanes end with the same result.
template <int PER, int LPT, int NSEL>
__device__ __forceinline__ void select_top(const float (&v)[PER], int q, int E, float (&sel_v)[NSEL],
                                           int (&sel_i)[NSEL]) {
  static_assert(PER <= 32, "one bit per owned expert");
  unsigned taken = 0;
#pragma unroll
  for (int r = 0; r < NSEL; r++) {
    float best = 0.f;
    int bi = kNone;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      const int e = q * PER + j;
      const bool ok = e < E && !((taken >> j) & 1u);
      if (ok && (bi == kNone || v[j] > best)) { best = v[j]; bi = e; }
    }
#pragma unroll
    for (int off = 1; off < LPT; off <<= 1) {
      const float ov = __shfl_xor(best, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      // the lower index is the incumbent; kNone is above every index
      const bool take = oi < bi ? !(bi != kNone && best > ov) : (oi != kNone && oi != bi && ov > best);
      if (take) { best = ov; bi = oi; }
    }
    sel_v[r] = best;
    sel_i[r] = bi;
    if (bi != kNone && bi / PER == q) taken |= 1u << (bi % PER);
  }
}

// run.cpp:336-354 with size = 4; v[0] is the maximum.
__device__ __forceinline__ float4 softmax4(const float (&v)[kTopK]) {
  const double mx = (double)v[0];
  float ev[kTopK];
  double sum = 0.0;
#pragma unroll
  for (int r = 0; r < kTopK; r++) {
    ev[r] = expf((float)((double)v[r] - mx));
    sum += (double)ev[r];
  }
  return make_float4((float)((double)ev[0] / sum), (float)((double)ev[1] / sum),
                     (float)((double)ev[2] / sum), (float)((double)ev[3] / sum));
}

// Top-NSEL of one token's logits for up to 32 experts, one lane per expert (the
// 32 lanes of a half wave; lane e owns expert e, v = its logit, -inf for a lane
// without an expert).  row4 points at the token's E_pad logits in LDS, 16-byte
// aligned.  Same rule as select_top, found by counting instead of five rounds
// of comparisons: an expert's place is the number of experts with a greater
// value; the lanes at places 0 .. NSEL-1 post themselves to `post` (LDS, NSEL
// floats then NSEL ints, owned by this token) and every lane reads the list
// back.  Of experts with equal values the lowest index takes the place (an
// atomic minimum) and the place behind it stays empty: an empty place among the
// first NSEL, like a NaN among the logits (which no count orders), sends the
// wave -- the branch is per wave -- through select_top's comparison-by-
// comparison rule instead.  Places past the number of experts hold kNone.
template <int E_pad, int NSEL>
__device__ __forceinline__ void ranked_top(const float4 *row4, float v, int e, int E, float *post,
                                           float (&sel_v)[NSEL], int (&sel_i)[NSEL]) {
  static_assert(E_pad == 16 || E_pad == 32, "one lane per expert in a half wave");
  int *post_i = reinterpret_cast<int *>(post + NSEL);
  if (e < NSEL) post_i[e] = kNone;
  int place = 0;
#pragma unroll
  for (int j4 = 0; j4 < E_pad / 4; j4++) {
    const float4 o = row4[j4];  // the same address in all lanes of the half wave
    place += (o.x > v ? 1 : 0) + (o.y > v ? 1 : 0) + (o.z > v ? 1 : 0) + (o.w > v ? 1 : 0);
  }
  if (e < E && place < NSEL) {
    post[place] = v;  // equal values: the same float from every writer
    atomicMin(&post_i[place], e);
  }
  // the same wave wrote the list; LDS operations of a wave complete in order
  bool redo = v != v;
#pragma unroll
  for (int r = 0; r < NSEL; r++) {
    sel_v[r] = post[r];
    sel_i[r] = post_i[r];
    redo |= r < E && sel_i[r] == kNone;
  }
  if (__ballot(redo) != 0ull) {
    const float own[1] = {v};
    select_top<1, 32, NSEL>(own, e, E, sel_v, sel_i);
  }
}

// The softmax of run.cpp:336-354 over the four selected logits with the work
// spread over four lanes of the token (lane r < 4 computes exp and quotient of
// place r; the sum is formed in every lane in the order of the reference), and
// the token's ids and weights stored by those lanes.  base = the token's first
// lane in the wave.
__device__ __forceinline__ void store_topk_spread(const float (&v)[kTopK], const int (&id)[kTopK], int r,
                                                  int base, int *topk_i_row, float *topk_v_row) {
  const double mx = (double)v[0];
  const float mine = r == 0 ? v[0] : (r == 1 ? v[1] : (r == 2 ? v[2] : v[3]));
  const float ev = expf((float)((double)mine - mx));
  double sum = 0.0;
#pragma unroll
  for (int k = 0; k < kTopK; k++) sum += (double)__shfl(ev, base + k, 64);
  if (r < kTopK) {
    topk_i_row[r] = r == 0 ? id[0] : (r == 1 ? id[1] : (r == 2 ? id[2] : id[3]));
    topk_v_row[r] = (float)((double)ev / sum);
  }
}

__device__ __forceinline__ void unpack8(const uint4 v, float (&f)[8]) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

// One workgroup = MT * 16 tokens x all experts (NT = E_pad / 16 blocks of 16).
// Its WPC waves split the reduction dimension in chunks of 32 (wave w takes
// chunks w, w + WPC, ...); D register sets of loads run ahead of the MFMAs.
// rstat[0] = max_e |w_e| (slightly inflated), rstat[1] = max_e |b_e|.
template <int NT, int WPC, int MT, int D, int FLUSH>
__global__ __launch_bounds__(WPC * 64) void router_kernel(
    const uint16_t *__restrict__ x, const int *__restrict__ pos, const uint16_t *__restrict__ wr,
    const float *__restrict__ br, const float *__restrict__ rstat, int T, int H, int E,
    float *__restrict__ score, int *__restrict__ topk_i, float *__restrict__ topk_v) {
  constexpr int E_pad = NT * 16;
  constexpr int TOK = MT * 16;
  // selection: LPT lanes per token, each owning PER experts; SW waves take part.
  // Up to 32 experts: one lane per expert, places found by counting (ranked_top).
  constexpr bool RANKED = E_pad <= 32;
  constexpr int LPT = RANKED ? 32 : (E_pad <= 64 ? 4 : (E_pad == 128 ? 8 : 16));
  constexpr int PER = RANKED ? 1 : E_pad / LPT;
  constexpr int SW = TOK * LPT / 64;
  static_assert(SW >= 1 && SW <= WPC, "waves of the selection");
  constexpr int LOG_LD = RANKED ? E_pad + 4 : E_pad + 1;  // RANKED reads rows of logits in 16-byte pieces
  // cross-wave sum: GB blocks of 16 x 16 outputs at a time through 32 KB
  constexpr int NBLK = MT * NT;
  constexpr int GB = 32 / WPC < NBLK ? 32 / WPC : NBLK;
  static_assert(WPC >= 2 && NBLK % GB == 0, "groups of the cross-wave sum");
  __shared__ double part[WPC / 2][GB][4][64];  // [wave][block][reg][lane]
  __shared__ float sumsq[WPC][TOK];
  __shared__ __attribute__((aligned(16))) float logits[TOK][LOG_LD];
  __shared__ float posted[RANKED ? TOK : 1][2 * (kTopK + 1)];  // ranked_top's lists
  __shared__ unsigned short tasks[TOK * E_pad];  // (token in tile) * E_pad + expert
  __shared__ int n_tasks;
  __shared__ float sh_br[E_pad];  // the bias, fetched while the first pass runs

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = tid >> 6;
  const int tok0 = blockIdx.x * TOK;
  const int row = lane & 15;  // token within a tile of 16 (first operand's row)
  const int g = lane >> 4;    // which 8 of the chunk's 32 k this lane holds
  const int kc_total = H / 32;
  if (tid == 0) n_tasks = 0;
  if (tid < E_pad) sh_br[tid] = br[tid];
  // the selection's own inputs, loaded long before they are needed
  const int tr = w * (64 / LPT) + lane / LPT;  // token within the workgroup (waves < SW only)
  const int q = lane % LPT;
  const int t = tok0 + tr;
  const bool active = w < SW && t < T && !(pos && pos[min(t, T - 1)] < 0);
  const float wn_max = rstat[0], bmax = rstat[1];

  f32x4 acc32[MT][NT], nrm[MT];
  double acc64[MT][NT][4];
#pragma unroll
  for (int m = 0; m < MT; m++) {
    nrm[m] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < NT; n++) {
      acc32[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < 4; i++) acc64[m][n][i] = 0.0;
    }
  }
  auto flush = [&]() {
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
      for (int n = 0; n < NT; n++) {
#pragma unroll
        for (int i = 0; i < 4; i++) acc64[m][n][i] += (double)acc32[m][n][i];
        acc32[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
  };

  const uint16_t *xrow[MT];
#pragma unroll
  for (int m = 0; m < MT; m++) xrow[m] = x + (size_t)min(tok0 + 16 * m + row, T - 1) * H + g * 8;
  const uint16_t *wlane = wr + (size_t)lane * 8;
  uint4 xs[D][MT], wq[D][NT];
  auto load = [&](int d, int c) {
    const int cc = min(c, kc_total - 1);  // only the first D loads of a wave can lie past the end
#pragma unroll
    for (int m = 0; m < MT; m++) xs[d][m] = *reinterpret_cast<const uint4 *>(xrow[m] + cc * 32);
#pragma unroll
    for (int n = 0; n < NT; n++)
      wq[d][n] = *reinterpret_cast<const uint4 *>(wlane + ((size_t)n * kc_total + cc) * 512);
  };
#pragma unroll
  for (int d = 0; d < D; d++) load(d, w + d * WPC);
  int since_flush = 0;
  for (int c0 = w; c0 < kc_total; c0 += D * WPC) {
#pragma unroll
    for (int d = 0; d < D; d++) {
      const int c = c0 + d * WPC;
      if (c < kc_total) {  // the same for the whole wave
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const bf16x8 xa = __builtin_bit_cast(bf16x8, xs[d][m]);
#pragma unroll
          for (int n = 0; n < NT; n++)
            acc32[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                xa, __builtin_bit_cast(bf16x8, wq[d][n]), acc32[m][n], 0, 0, 0);
          nrm[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, xa, nrm[m], 0, 0, 0);
        }
        if (c + D * WPC < kc_total) load(d, c + D * WPC);  // nothing is loaded that is not used
        if (FLUSH == 1 || ++since_flush == FLUSH) {
          flush();
          since_flush = 0;
        }
      }
    }
  }
  flush();

  // |x_t|^2 is the diagonal of x x^T: register i of lane l is (row 4*(l/16) + i,
  // column l % 16).
  if ((row >> 2) == g) {
#pragma unroll
    for (int m = 0; m < MT; m++) {
      const int i = row & 3;
      sumsq[w][16 * m + row] = i == 0 ? nrm[m][0] : (i == 1 ? nrm[m][1] : (i == 2 ? nrm[m][2] : nrm[m][3]));
    }
  }
  // The waves' fp64 sums are added up in a fixed order (the same sum in every
  // run): the upper half of the waves hands its sums to the lower half, whose
  // results all threads then add in wave order; GB blocks at a time.
#pragma unroll
  for (int b0 = 0; b0 < NBLK; b0 += GB) {
    if (w >= WPC / 2) {
#pragma unroll
      for (int b = 0; b < GB; b++)
#pragma unroll
        for (int i = 0; i < 4; i++) part[w - WPC / 2][b][i][lane] = acc64[(b0 + b) / NT][(b0 + b) % NT][i];
    }
    __syncthreads();
    if (w < WPC / 2) {
#pragma unroll
      for (int b = 0; b < GB; b++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          part[w][b][i][lane] += acc64[(b0 + b) / NT][(b0 + b) % NT][i];
    }
    __syncthreads();
    // Register i of lane l is token 4*(l/16) + i of its tile, expert 16*n + l%16.
    for (int idx = tid; idx < GB * 256; idx += WPC * 64) {
      const int l = idx & 63;
      const int i = (idx >> 6) & 3;
      const int b = b0 + (idx >> 8);
      const int m = b / NT, n = b % NT;
      const int e = 16 * n + (l & 15);
      double sd = 0.0;
#pragma unroll
      for (int ww = 0; ww < WPC / 2; ww++) sd += part[ww][idx >> 8][i][l];
      float f = (float)sd;  // run.cpp:368
      f += sh_br[e];        // run.cpp:669-671
      logits[16 * m + 4 * (l >> 4) + i][e] = f;
    }
    __syncthreads();
  }

  // Pass 2, selection: LPT lanes per token.
  bool undecided = false;
  if (w < SW) {
    float v[PER];
    float s_v[kTopK + 1];
    int s_i[kTopK + 1];
    if constexpr (RANKED) {
      v[0] = q < E_pad ? logits[tr][q] : -__builtin_inff();
      ranked_top<E_pad, kTopK + 1>(reinterpret_cast<const float4 *>(&logits[tr][0]), v[0], q, E, posted[tr],
                                   s_v, s_i);
    } else {
#pragma unroll
      for (int j = 0; j < PER; j++) v[j] = logits[tr][q * PER + j];
      select_top<PER, LPT, kTopK + 1>(v, q, E, s_v, s_i);
    }
    if (active) {
      float ss = 0.f;
#pragma unroll
      for (int ww = 0; ww < WPC; ww++) ss += sumsq[ww][tr];
      // bound on |first-pass logit - exact logit|: the accumulation error plus
      // the two float roundings (sum -> float, + bias) of either arithmetic
      const float err0 = router_gamma(FLUSH) * sqrtf(ss * 1.002f) * wn_max;
      auto up = [&](float a) { return a + (4.76837158e-7f * (fabsf(a) + bmax) + err0); };
      auto lo = [&](float a) { return a - (4.76837158e-7f * (fabsf(a) + bmax) + err0); };
      const bool decided = lo(s_v[0]) > up(s_v[1]) && lo(s_v[1]) > up(s_v[2]) && lo(s_v[2]) > up(s_v[3]) &&
                           (s_i[4] == kNone || lo(s_v[3]) > up(s_v[4]));
      if (decided) {
        if constexpr (RANKED) {
          // (tokens of one wave can differ in `decided`: the shuffles inside are
          // among the lanes of one token, which agree)
          const float sv[kTopK] = {s_v[0], s_v[1], s_v[2], s_v[3]};
          const int si[kTopK] = {s_i[0], s_i[1], s_i[2], s_i[3]};
          store_topk_spread(sv, si, q, lane - q, topk_i + (size_t)t * kTopK, topk_v + (size_t)t * kTopK);
        } else if (q == 0) {
          const float sv[kTopK] = {s_v[0], s_v[1], s_v[2], s_v[3]};
          *reinterpret_cast<int4 *>(topk_i + (size_t)t * kTopK) = make_int4(s_i[0], s_i[1], s_i[2], s_i[3]);
          *reinterpret_cast<float4 *>(topk_v + (size_t)t * kTopK) = softmax4(sv);
        }
      } else {
        undecided = true;
        // contenders: everything not provably below the fourth best (a NaN
        // anywhere makes the comparison fail, and the expert a contender)
        const float floor4 = lo(s_v[3]);
#pragma unroll
        for (int j = 0; j < PER; j++) {
          const int e = q * PER + j;
          if (e < E && !(up(v[j]) < floor4)) tasks[atomicAdd(&n_tasks, 1)] = (unsigned short)(tr * E_pad + e);
        }
      }
    } else if (t < T && q == 0) {
      *reinterpret_cast<int4 *>(topk_i + (size_t)t * kTopK) = make_int4(-1, -1, -1, -1);
      *reinterpret_cast<float4 *>(topk_v + (size_t)t * kTopK) = make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  __syncthreads();

  // Exact logits of the contenders, one wave per (token, expert): float
  // products, fp64 sum, one rounding to float, bias added in float.  A wave
  // takes TPW tasks at a time and has all their loads in flight at once (the
  // phase is a chain of memory round trips otherwise).
  constexpr int TPW = WPC >= 8 ? 1 : 2;
  constexpr int PIECES = 6;  // 16-byte pieces per lane and operand in one round: 3072 k
  const int nt = n_tasks;
  const int n_pieces = H / 8;
  for (int task0 = w * TPW; task0 < nt; task0 += WPC * TPW) {
    double s[TPW];
    const uint16_t *xr[TPW], *we[TPW];
    int tt[TPW], ee[TPW];
#pragma unroll
    for (int j = 0; j < TPW; j++) {
      const int code = tasks[min(task0 + j, nt - 1)];
      tt[j] = code / E_pad;
      ee[j] = code % E_pad;
      xr[j] = x + (size_t)min(tok0 + tt[j], T - 1) * H;
      we[j] = wr + ((size_t)(ee[j] >> 4) * kc_total * 64 + (ee[j] & 15)) * 8;
      s[j] = 0.0;
    }
    for (int p0 = 0; p0 < n_pieces; p0 += 64 * PIECES) {
      uint4 xv[TPW][PIECES], wv[TPW][PIECES];
#pragma unroll
      for (int j = 0; j < TPW; j++)
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
          // piece p: k = 8p .. 8p+7 = chunk p/4, quarter p%4; past the row's end: piece 0, not used
          const int pp = p0 + i * 64 + lane;
          const int p = pp < n_pieces ? pp : 0;
          xv[j][i] = *reinterpret_cast<const uint4 *>(xr[j] + p * 8);
          wv[j][i] = *reinterpret_cast<const uint4 *>(we[j] + ((size_t)(p >> 2) * 64 + (p & 3) * 16) * 8);
        }
#pragma unroll
      for (int j = 0; j < TPW; j++)
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
          if (p0 + i * 64 + lane < n_pieces) {
            float xf[8], wf[8];
            unpack8(xv[j][i], xf);
            unpack8(wv[j][i], wf);
#pragma unroll
            for (int k = 0; k < 8; k++) s[j] += (double)(xf[k] * wf[k]);
          }
        }
    }
#pragma unroll
    for (int j = 0; j < TPW; j++) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) s[j] += __shfl_xor(s[j], off, 64);
      if (lane == 0 && task0 + j < nt) {
        float f = (float)s[j];
        f += sh_br[ee[j]];
        logits[tt[j]][ee[j]] = f;
      }
    }
  }
  __syncthreads();

  if constexpr (RANKED) {
    if (w < SW && __ballot(undecided) != 0ull) {  // per wave: ranked_top is a wave's work
      const float v = q < E_pad ? logits[tr][q] : -__builtin_inff();
      float s_v[kTopK];
      int s_i[kTopK];
      ranked_top<E_pad, kTopK>(reinterpret_cast<const float4 *>(&logits[tr][0]), v, q, E, posted[tr], s_v, s_i);
      if (undecided) store_topk_spread(s_v, s_i, q, lane - q, topk_i + (size_t)t * kTopK, topk_v + (size_t)t * kTopK);
    }
  } else if (undecided) {  // waves < SW only
    float v[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) v[j] = logits[tr][q * PER + j];
    float s_v[kTopK];
    int s_i[kTopK];
    select_top<PER, LPT, kTopK>(v, q, E, s_v, s_i);
    if (q == 0) {
      *reinterpret_cast<int4 *>(topk_i + (size_t)t * kTopK) = make_int4(s_i[0], s_i[1], s_i[2], s_i[3]);
      *reinterpret_cast<float4 *>(topk_v + (size_t)t * kTopK) = softmax4(s_v);
    }
  }
  if (score) {
    for (int idx = tid; idx < TOK * E_pad; idx += WPC * 64) {
      const int tt = idx / E_pad, e = idx % E_pad;
      const int ts = tok0 + tt;
      if (e < E && ts < T && !(pos && pos[ts] < 0)) score[(size_t)ts * E + e] = logits[tt][e];
    }
  }
}

// Statistics of a layer's router for the error bound of the first pass:
// rstat[0] = max_e |w_e|_2 over the bf16-rounded weights (inflated by 1e-3 for
// the rounding of this very sum), rstat[1] = max_e |b_e|.  One workgroup.
__global__ __launch_bounds__(256) void router_stats_kernel(const float *__restrict__ w,
                                                           const float *__restrict__ b, int E, int H,
                                                           float *__restrict__ rstat) {
  __shared__ float red[256];
  float wmax = 0.f, bmax = 0.f;
  for (int e = 0; e < E; e++) {
    float s = 0.f;
    for (int k = threadIdx.x; k < H; k += 256) {
      const float v = __uint_as_float((uint32_t)f32_to_bf16_rne(w[(size_t)e * H + k]) << 16);
      s += v * v;
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
      if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
      __syncthreads();
    }
    wmax = fmaxf(wmax, red[0]);
    __syncthreads();
    bmax = fmaxf(bmax, fabsf(__uint_as_float((uint32_t)f32_to_bf16_rne(b[e]) << 16)));
  }
  if (threadIdx.x == 0) {
    rstat[0] = sqrtf(wmax) * 1.001f;
    rstat[1] = bmax;
  }
}

hipError_t launch_router_stats(const float *w_src, const float *b_src, int E, int H, float *rstat,
                               hipStream_t s) {
  router_stats_kernel<<<1, 256, 0, s>>>(w_src, b_src, E, H, rstat);
  return hipGetLastError();
}

template <int NT>
static hipError_t launch_router_nt(const uint16_t *x, const int *pos, const uint16_t *wr,
                                   const float *br, const float *rstat, int T, int H, int E,
                                   float *score, int *topk_i, float *topk_v, hipStream_t s) {
  // As fine a split of the reduction as the registers allow: more waves keep
  // more loads in flight, and small batches still occupy the SIMDs.  D register
  // sets of 4 * (MT + NT) registers each run ahead.
  constexpr int WPC = NT <= 2 ? 16 : (NT <= 4 ? 8 : 4);
  constexpr int D = NT <= 2 ? 6 : (NT <= 4 ? 4 : (NT <= 8 ? 3 : 2));
  // MFMAs between two hand-overs to fp64: the fewer, the tighter the bound and
  // the fewer tokens take the second pass, at 8 * NT more fp64 instructions
  // each; the first pass is bound by its loads, so the hand-over after every
  // MFMA costs nothing
  constexpr int FLUSH = 1;
  // Every workgroup streams the whole router matrix through its CU; at 128
  // experts a workgroup takes two tiles of 16 tokens so that half as many do
  // (at 256 the accumulators of two tiles no longer fit the registers).
  if (NT == 8 && T > 256 * 16) {
    constexpr int MT = NT == 8 ? 2 : 1;
    router_kernel<NT, WPC, MT, D, FLUSH><<<(T + 16 * MT - 1) / (16 * MT), WPC * 64, 0, s>>>(
        x, pos, wr, br, rstat, T, H, E, score, topk_i, topk_v);
  } else {
    router_kernel<NT, WPC, 1, D, FLUSH><<<(T + 15) / 16, WPC * 64, 0, s>>>(x, pos, wr, br, rstat, T, H, E,
                                                                          score, topk_i, topk_v);
  }
  return hipGetLastError();
}

hipError_t launch_router(const uint16_t *x, const int *pos, const uint16_t *wr, const float *br,
                         const float *rstat, int T, int H, int E, int E_pad, float *score, int *topk_i,
                         float *topk_v, hipStream_t s) {
  if (T <= 0) return hipSuccess;
  switch (E_pad / 16) {
    case 1: return launch_router_nt<1>(x, pos, wr, br, rstat, T, H, E, score, topk_i, topk_v, s);
    case 2: return launch_router_nt<2>(x, pos, wr, br, rstat, T, H, E, score, topk_i, topk_v, s);
    case 4: return launch_router_nt<4>(x, pos, wr, br, rstat, T, H, E, score, topk_i, topk_v, s);
    case 8: return launch_router_nt<8>(x, pos, wr, br, rstat, T, H, E, score, topk_i, topk_v, s);
    case 16: return launch_router_nt<16>(x, pos, wr, br, rstat, T, H, E, score, topk_i, topk_v, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe
