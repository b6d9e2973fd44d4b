// RMS normalisation in front of the layer.  Replaces rmsnorm_batch_kernel
// (utility/utility.cpp:194-271; call getp_run.cpp:688-695) with the arithmetic of
// the CPU path (run.cpp:321-334): squares are exact in fp32 for bf16 inputs and
// are summed in fp64, the scale 1/sqrt(mean + 1e-5) is formed in fp32 with
// correctly rounded sqrt and division, the product weight * (scale * x) is
// rounded once to fp32 and then to bf16, the layer's input type.  The one
// difference from a sequential sum is the order of the fp64 additions, which
// reaches the fp32 scale only where two fp64 sums that differ in their last bit
// straddle an fp32 rounding boundary.
#include "moe_internal.h"

namespace moe {

// One wave per token, 8 elements (16 bytes) per lane and pass.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t *__restrict__ x,
                                                     const float *__restrict__ weight,
                                                     const int *__restrict__ pos,
                                                     uint16_t *__restrict__ t_out, int T, int H) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  if (pos && pos[t] < 0) return;  // the row takes part in nothing downstream
  const uint4 *row = reinterpret_cast<const uint4 *>(x + (size_t)t * H);
  const int chunks = H / 8;
  double ss = 0.0;
  for (int c = lane; c < chunks; c += 64) {
    const uint4 v = row[c];
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float a = __uint_as_float(u[i] << 16), b = __uint_as_float(u[i] & 0xffff0000u);
      ss += (double)(a * a);
      ss += (double)(b * b);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
  ss /= (double)H;
  ss += (double)1e-5f;
  const float narrowed = (float)ss;
  const float root = (float)sqrt((double)narrowed);  // = sqrtf, correctly rounded
  const float scale = (float)(1.0 / (double)root);    // = 1.0f / root, correctly rounded
  uint4 *out = reinterpret_cast<uint4 *>(t_out + (size_t)t * H);
  for (int c = lane; c < chunks; c += 64) {
    const uint4 v = row[c];
    const float4 w0 = *reinterpret_cast<const float4 *>(weight + 8 * c);
    const float4 w1 = *reinterpret_cast<const float4 *>(weight + 8 * c + 4);
    const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float a = __uint_as_float(u[i] << 16), b = __uint_as_float(u[i] & 0xffff0000u);
      const float ra = (float)((double)w[2 * i] * ((double)scale * (double)a));
      const float rb = (float)((double)w[2 * i + 1] * ((double)scale * (double)b));
      o[i] = f32_to_bf16_rne(ra) | ((uint32_t)f32_to_bf16_rne(rb) << 16);
    }
    out[c] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// Rows of H bf16 values copied into rows of Hp >= H, the rest zero: the grouped
// GEMMs reduce over multiples of 64, and a hidden size that is not one (the
// reference's 7M model has 32, export_model_bin/gpt-oss-7m/config.json:3) is
// widened here, once per call, rather than read past the end of its rows.
__global__ __launch_bounds__(256) void pad_rows_kernel(const uint4 *__restrict__ x, uint4 *__restrict__ xp,
                                                      int T, int H8, int Hp8) {
  const size_t n = (size_t)T * Hp8;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    const size_t t = i / Hp8;
    const int c = (int)(i % Hp8);
    xp[i] = c < H8 ? x[t * H8 + c] : make_uint4(0u, 0u, 0u, 0u);
  }
}

hipError_t launch_pad_rows(const uint16_t *x, uint16_t *xp, int T, int H, int Hp, hipStream_t s) {
  const size_t n = (size_t)T * (Hp / 8);
  const int grid = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  pad_rows_kernel<<<grid, 256, 0, s>>>(reinterpret_cast<const uint4 *>(x), reinterpret_cast<uint4 *>(xp), T,
                                       H / 8, Hp / 8);
  return hipGetLastError();
}

hipError_t launch_rmsnorm(const uint16_t *x, const float *weight, const int *pos, uint16_t *t_out,
                          int T, int H, hipStream_t s) {
  rmsnorm_kernel<<<(T + 3) / 4, 256, 0, s>>>(x, weight, pos, t_out, T, H);
  return hipGetLastError();
}

}  // namespace moe
