// Router: logits = x * Wr^T + br, top-4 with ties to the lower expert id,
// softmax over the four selected logits.  Replaces matmul_router_kernel
// (matmul/matmul.cpp:945-1019) and fused_topk_softmax_batch_kernel
// (utility/utility.cpp:273-365); the arithmetic follows the reference's CPU path
// (run.cpp:356-369 matmul, :388-421 topk, :336-354 softmax) so that the expert
// ids are reproduced exactly:
//   * products of two bf16 values are exact in fp32; they are accumulated in
//     fp64 on the matrix cores (v_mfma_f64_16x16x4_f64), as run.cpp:363-367
//     accumulates float products in a double; the sum is rounded to float once
//     and the bias is added in float (run.cpp:669-671);
//   * the top-4 comparison is (value descending, index ascending);
//   * the softmax keeps the sum in double and divides in double.
#include "moe_internal.h"

namespace moe {

typedef double f64x4 __attribute__((ext_vector_type(4)));

// One workgroup = 16 tokens x all experts.  Its WPC waves split the reduction
// dimension in chunks of 32 (wave w takes chunks w, w+WPC, ...), each wave
// keeps NT 16x16 accumulators, and the partial sums are added in wave order
// through LDS.  NT = E_pad / 16.
template <int NT, int WPC>
__global__ __launch_bounds__(WPC * 64) void router_kernel(
    const uint16_t *__restrict__ x, const int *__restrict__ pos, const double *__restrict__ wr,
    const float *__restrict__ br, int T, int H, int E, float *__restrict__ score,
    int *__restrict__ topk_i, float *__restrict__ topk_v) {
  constexpr int E_pad = NT * 16;
  __shared__ double part[WPC][NT][4][64];  // [wave][expert block][reg][lane]
  __shared__ float logits[16][E_pad + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = tid >> 6;
  const int tok0 = blockIdx.x * 16;
  const int row = lane & 15;  // token within the tile (A-operand row)
  const int g = lane >> 4;    // which 8 of the chunk's 32 k this lane holds
  const int t_ld = min(tok0 + row, T - 1);
  const int kc_total = H / 32;

  f64x4 acc[NT];
#pragma unroll
  for (int n = 0; n < NT; n++) acc[n] = f64x4{0.0, 0.0, 0.0, 0.0};

  const uint16_t *xrow = x + (size_t)t_ld * H + g * 8;
  for (int c = w; c < kc_total; c += WPC) {
    const uint4 xv = *reinterpret_cast<const uint4 *>(xrow + c * 32);
    double xd[8];
    xd[0] = (double)__uint_as_float(xv.x << 16);
    xd[1] = (double)__uint_as_float(xv.x & 0xffff0000u);
    xd[2] = (double)__uint_as_float(xv.y << 16);
    xd[3] = (double)__uint_as_float(xv.y & 0xffff0000u);
    xd[4] = (double)__uint_as_float(xv.z << 16);
    xd[5] = (double)__uint_as_float(xv.z & 0xffff0000u);
    xd[6] = (double)__uint_as_float(xv.w << 16);
    xd[7] = (double)__uint_as_float(xv.w & 0xffff0000u);
#pragma unroll
    for (int n = 0; n < NT; n++) {
      const double *wp = wr + (((size_t)n * kc_total + c) * 64 + lane) * 8;
      const double2 w01 = *reinterpret_cast<const double2 *>(wp);
      const double2 w23 = *reinterpret_cast<const double2 *>(wp + 2);
      const double2 w45 = *reinterpret_cast<const double2 *>(wp + 4);
      const double2 w67 = *reinterpret_cast<const double2 *>(wp + 6);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[0], w01.x, acc[n], 0, 0, 0);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[1], w01.y, acc[n], 0, 0, 0);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[2], w23.x, acc[n], 0, 0, 0);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[3], w23.y, acc[n], 0, 0, 0);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[4], w45.x, acc[n], 0, 0, 0);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[5], w45.y, acc[n], 0, 0, 0);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[6], w67.x, acc[n], 0, 0, 0);
      acc[n] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[7], w67.y, acc[n], 0, 0, 0);
    }
  }

#pragma unroll
  for (int n = 0; n < NT; n++) {
#pragma unroll
    for (int i = 0; i < 4; i++) part[w][n][i][lane] = acc[n][i];
  }
  __syncthreads();

  // Result register i of lane l is token 4*i + l/16, expert 16*n + l%16.
  for (int idx = tid; idx < NT * 4 * 64; idx += WPC * 64) {
    const int l = idx & 63;
    const int i = (idx >> 6) & 3;
    const int n = idx >> 8;
    double s = 0.0;
#pragma unroll
    for (int ww = 0; ww < WPC; ww++) s += part[ww][n][i][l];
    const int e = 16 * n + (l & 15);
    const int tr = 4 * i + (l >> 4);
    float f = (float)s;  // run.cpp:368
    f += br[e];          // run.cpp:669-671
    logits[tr][e] = f;
    const int t = tok0 + tr;
    if (score && e < E && t < T && !(pos && pos[t] < 0)) score[(size_t)t * E + e] = f;
  }
  __syncthreads();

  if (w != 0) return;
  // Wave 0: four lanes per token, each owning a contiguous quarter of the experts.
  constexpr int PER = E_pad / 4;
  const int tr = lane >> 2;
  const int q = lane & 3;
  float v[PER];
#pragma unroll
  for (int j = 0; j < PER; j++) v[j] = logits[tr][q * PER + j];

  float sel_v[kTopK];
  int sel_i[kTopK];
#pragma unroll
  for (int r = 0; r < kTopK; r++) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      if (v[j] > best) { best = v[j]; bi = q * PER + j; }
    }
#pragma unroll
    for (int off = 1; off < 4; off <<= 1) {
      const float ov = __shfl_xor(best, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    sel_v[r] = best;
    sel_i[r] = bi;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      if (q * PER + j == bi) v[j] = -INFINITY;
    }
  }

  const int t = tok0 + tr;
  if (q != 0 || t >= T) return;
  int4 oi;
  float4 ov;
  if (pos && pos[t] < 0) {
    oi = make_int4(-1, -1, -1, -1);
    ov = make_float4(0.f, 0.f, 0.f, 0.f);
  } else {
    // run.cpp:336-354 with size = 4; sel_v[0] is the maximum.
    const double mx = (double)sel_v[0];
    float ev[kTopK];
    double sum = 0.0;
#pragma unroll
    for (int r = 0; r < kTopK; r++) {
      ev[r] = expf((float)((double)sel_v[r] - mx));
      sum += (double)ev[r];
    }
    oi = make_int4(sel_i[0], sel_i[1], sel_i[2], sel_i[3]);
    ov = make_float4((float)((double)ev[0] / sum), (float)((double)ev[1] / sum),
                     (float)((double)ev[2] / sum), (float)((double)ev[3] / sum));
  }
  *reinterpret_cast<int4 *>(topk_i + (size_t)t * kTopK) = oi;
  *reinterpret_cast<float4 *>(topk_v + (size_t)t * kTopK) = ov;
}

template <int NT>
static hipError_t launch_router_nt(const uint16_t *x, const int *pos, const double *wr,
                                   const float *br, int T, int H, int E, float *score, int *topk_i,
                                   float *topk_v, hipStream_t s) {
  const int grid = (T + 15) / 16;
  // More waves per workgroup (a finer split of the reduction) when there are
  // too few token tiles to occupy the 1024 SIMDs; bounded by the LDS the
  // partial sums need (WPC * NT * 2 KB).
  if constexpr (NT <= 2) {
    if (grid < 128) {
      router_kernel<NT, 16><<<grid, 16 * 64, 0, s>>>(x, pos, wr, br, T, H, E, score, topk_i, topk_v);
      return hipGetLastError();
    }
  }
  if constexpr (NT <= 4) {
    if (grid < 256) {
      router_kernel<NT, 8><<<grid, 8 * 64, 0, s>>>(x, pos, wr, br, T, H, E, score, topk_i, topk_v);
      return hipGetLastError();
    }
  }
  router_kernel<NT, 4><<<grid, 4 * 64, 0, s>>>(x, pos, wr, br, T, H, E, score, topk_i, topk_v);
  return hipGetLastError();
}

hipError_t launch_router(const uint16_t *x, const int *pos, const double *wr, const float *br, int T,
                         int H, int E, int E_pad, float *score, int *topk_i, float *topk_v,
                         hipStream_t s) {
  if (T <= 0) return hipSuccess;
  switch (E_pad / 16) {
    case 1: return launch_router_nt<1>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, s);
    case 2: return launch_router_nt<2>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, s);
    case 4: return launch_router_nt<4>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, s);
    case 8: return launch_router_nt<8>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, s);
    case 16: return launch_router_nt<16>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe
