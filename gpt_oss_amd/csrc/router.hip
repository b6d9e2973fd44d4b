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

// 8 bf16 -> 8 doubles (exact).
__device__ __forceinline__ void widen8(const uint4 v, double (&d)[8]) {
  d[0] = (double)__uint_as_float(v.x << 16);
  d[1] = (double)__uint_as_float(v.x & 0xffff0000u);
  d[2] = (double)__uint_as_float(v.y << 16);
  d[3] = (double)__uint_as_float(v.y & 0xffff0000u);
  d[4] = (double)__uint_as_float(v.z << 16);
  d[5] = (double)__uint_as_float(v.z & 0xffff0000u);
  d[6] = (double)__uint_as_float(v.w << 16);
  d[7] = (double)__uint_as_float(v.w & 0xffff0000u);
}

// One workgroup = 16 tokens x all experts.  Its WPC waves split the reduction
// dimension in chunks of 32 (wave w takes chunks w, w+WPC, ...), each wave
// keeps NT 16x16 accumulators, and the partial sums are added in wave order
// through LDS.  NT = E_pad / 16.
//
// SPLIT (small batches: a handful of workgroups would otherwise carry all the
// fp64 MFMAs on as many CUs, 20 us whatever the batch): gridDim.y workgroups
// share a tile of 16 tokens, each taking `cps` consecutive chunks.  They leave
// their sums in `ws`; the one that arrives last (a counter per tile) adds them
// up in the order of the chunks -- the same sum whichever arrives last -- and
// selects.  No workgroup waits for another.
template <int NT, int WPC, int D, bool SPLIT>
__global__ __launch_bounds__(WPC * 64) void router_kernel(
    const uint16_t *__restrict__ x, const int *__restrict__ pos, const uint16_t *__restrict__ wr,
    const float *__restrict__ br, int T, int H, int E, float *__restrict__ score,
    int *__restrict__ topk_i, float *__restrict__ topk_v, double *ws, int *arrivals, int cps) {
  constexpr int E_pad = NT * 16;
  __shared__ double part[WPC][NT][4][64];  // [wave][expert block][reg][lane]
  __shared__ float logits[16][E_pad + 1];
  __shared__ int is_last;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = tid >> 6;
  const int tok0 = blockIdx.x * 16;
  const int row = lane & 15;  // token within the tile (A-operand row)
  const int g = lane >> 4;    // which 8 of the chunk's 32 k this lane holds
  const int t_ld = min(tok0 + row, T - 1);
  const int kc_total = H / 32;
  const int c_begin = SPLIT ? (int)blockIdx.y * cps : 0;
  const int c_end = SPLIT ? min(c_begin + cps, kc_total) : kc_total;

  f64x4 acc[NT];
#pragma unroll
  for (int n = 0; n < NT; n++) acc[n] = f64x4{0.0, 0.0, 0.0, 0.0};

  // The wave's loads run D chunks ahead of its MFMAs (a ring of D register
  // sets): with few waves per SIMD nothing else covers their latency, and a
  // small batch is a handful of workgroups whose time is the chain of these
  // round trips.  Past the end the ring re-loads the last chunk and drops it.
  const uint16_t *xrow = x + (size_t)t_ld * H + g * 8;
  const uint16_t *wlane = wr + (size_t)lane * 8;
  uint4 xs[D], wq[D][NT];
  auto load = [&](int d, int c) {
    const int cc = min(c, c_end - 1);
    xs[d] = *reinterpret_cast<const uint4 *>(xrow + cc * 32);
#pragma unroll
    for (int n = 0; n < NT; n++)
      wq[d][n] = *reinterpret_cast<const uint4 *>(wlane + ((size_t)n * kc_total + cc) * 512);
  };
#pragma unroll
  for (int d = 0; d < D; d++) load(d, c_begin + w + d * WPC);
  for (int c0 = c_begin + w; c0 < c_end; c0 += D * WPC) {
#pragma unroll
    for (int d = 0; d < D; d++) {
      const int c = c0 + d * WPC;
      if (c < c_end) {  // the same for the whole wave
        double xd[8];
        widen8(xs[d], xd);
        // Two accumulators are advanced alternately so that back-to-back MFMAs do
        // not depend on each other.
        constexpr int NP = NT > 1 ? 2 : 1;
#pragma unroll
        for (int n = 0; n < NT; n += NP) {
          double wd[NP][8];
#pragma unroll
          for (int p = 0; p < NP; p++) widen8(wq[d][n + p], wd[p]);
#pragma unroll
          for (int s = 0; s < 8; s++)
#pragma unroll
            for (int p = 0; p < NP; p++)
              acc[n + p] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[s], wd[p][s], acc[n + p], 0, 0, 0);
        }
        load(d, c + D * WPC);
      }
    }
  }

#pragma unroll
  for (int n = 0; n < NT; n++) {
#pragma unroll
    for (int i = 0; i < 4; i++) part[w][n][i][lane] = acc[n][i];
  }
  __syncthreads();

  if (SPLIT) {
    const int S = gridDim.y;
    double *mine = ws + ((size_t)blockIdx.x * S + blockIdx.y) * (NT * 256);
    for (int idx = tid; idx < NT * 4 * 64; idx += WPC * 64) {
      double s = 0.0;
#pragma unroll
      for (int ww = 0; ww < WPC; ww++) s += (&part[ww][0][0][0])[idx];
      mine[idx] = s;
    }
    __threadfence();  // the sums are out before the arrival is counted
    __syncthreads();
    if (tid == 0) is_last = atomicAdd(&arrivals[blockIdx.x], 1) == S - 1;
    __syncthreads();
    if (!is_last) return;
    __threadfence();  // and the other workgroups' sums are read after it
  }

  // Result register i of lane l is token 4*i + l/16, expert 16*n + l%16.
  for (int idx = tid; idx < NT * 4 * 64; idx += WPC * 64) {
    const int l = idx & 63;
    const int i = (idx >> 6) & 3;
    const int n = idx >> 8;
    double s = 0.0;
    if (SPLIT) {
      // all loads first (they are independent), then the sum in chunk order
      const int S = gridDim.y;
      const double *all = ws + (size_t)blockIdx.x * S * (NT * 256) + idx;
      double v[kRouterSplitMax];
#pragma unroll
      for (int sp = 0; sp < kRouterSplitMax; sp++) v[sp] = sp < S ? all[(size_t)sp * (NT * 256)] : 0.0;
#pragma unroll
      for (int sp = 0; sp < kRouterSplitMax; sp++) s += v[sp];
    } else {
#pragma unroll
      for (int ww = 0; ww < WPC; ww++) s += part[ww][n][i][l];
    }
    const int e = 16 * n + (l & 15);
    const int tr = 4 * i + (l >> 4);
    float f = (float)s;  // run.cpp:368
    f += br[e];          // run.cpp:669-671
    logits[tr][e] = f;
    const int t = tok0 + tr;
    if (score && e < E && t < T && !(pos && pos[t] < 0)) score[(size_t)t * E + e] = f;
  }
  __syncthreads();
  if (SPLIT && tid == 0) arrivals[blockIdx.x] = 0;  // for the next launch

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

// Chunks of 32 k per workgroup when a tile of 16 tokens is shared (0: no
// sharing): batches of few tiles only, and never more than kRouterSplitMax
// workgroups per tile.
static int router_split_chunks(int T, int H) {
  const int tiles = (T + 15) / 16;
  const int kc_total = H / 32;
  if (tiles > kRouterSplitTiles) return 0;
  const int cps = (kc_total + kRouterSplitMax - 1) / kRouterSplitMax;
  return cps >= kc_total ? 0 : cps;
}

template <int NT>
static hipError_t launch_router_nt(const uint16_t *x, const int *pos, const uint16_t *wr,
                                   const float *br, int T, int H, int E, float *score, int *topk_i,
                                   float *topk_v, double *ws, int *arrivals, hipStream_t s) {
  const int grid = (T + 15) / 16;
  // Register sets in flight per wave, 4 * (1 + NT) registers each, within the
  // 128 / 256 / 512 registers a wave of a workgroup this size can have.
  constexpr int D = NT <= 2 ? 6 : (NT <= 4 ? 4 : (NT <= 8 ? 3 : 2));
  const int cps = ws ? router_split_chunks(T, H) : 0;
  if (cps > 0) {
    constexpr int WPS = NT <= 8 ? 4 : 2;  // waves of a workgroup that shares a tile
    constexpr int DS = D < 3 ? D : 3;
    const int S = (H / 32 + cps - 1) / cps;
    router_kernel<NT, WPS, DS, true><<<dim3(grid, S), WPS * 64, 0, s>>>(x, pos, wr, br, T, H, E, score, topk_i,
                                                                        topk_v, ws, arrivals, cps);
    return hipGetLastError();
  }
  // As many waves per workgroup (i.e. as fine a split of the reduction) as the
  // LDS for the partial sums allows (WPC * NT * 2 KB <= 64 KB): more waves per
  // SIMD hide the load latency, and small batches still occupy the SIMDs.
  constexpr int WPC = NT <= 2 ? 16 : (NT <= 4 ? 8 : (NT <= 8 ? 4 : 2));
  router_kernel<NT, WPC, D, false><<<grid, WPC * 64, 0, s>>>(x, pos, wr, br, T, H, E, score, topk_i,
                                                             topk_v, nullptr, nullptr, 0);
  return hipGetLastError();
}

hipError_t launch_router(const uint16_t *x, const int *pos, const uint16_t *wr, const float *br, int T,
                         int H, int E, int E_pad, float *score, int *topk_i, float *topk_v,
                         double *ws, int *arrivals, hipStream_t s) {
  if (T <= 0) return hipSuccess;
  switch (E_pad / 16) {
    case 1: return launch_router_nt<1>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, ws, arrivals, s);
    case 2: return launch_router_nt<2>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, ws, arrivals, s);
    case 4: return launch_router_nt<4>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, ws, arrivals, s);
    case 8: return launch_router_nt<8>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, ws, arrivals, s);
    case 16: return launch_router_nt<16>(x, pos, wr, br, T, H, E, score, topk_i, topk_v, ws, arrivals, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe
