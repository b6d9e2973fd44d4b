// Measured denominators for the rooflines the benchmark reports: what THIS GPU
// sustains on the instruction the grouped GEMMs are built from, and on a plain
// stream through HBM.  The published peaks (2.5 PFLOP/s dense bf16 at the
// nominal clock, 8 TB/s) are quoted next to them; these say how much of the
// distance to those is the kernels' and how much is the machine's.  They play
// the part of the reference's own tuning harness
// (getp-csrc/matmul/tune.cpp:1347-1595, results in matmul/log.txt), which times
// its kernels against each other but never against the hardware.
//
// Nothing here is used by the layer; the entry points allocate and free their
// own buffers and synchronise with the host.
#include "moe_internal.h"

namespace moe {
namespace {

typedef __bf16 ybf16x8 __attribute__((ext_vector_type(8)));
typedef float yf32x16 __attribute__((ext_vector_type(16)));

// 4 waves per workgroup, one per SIMD, each with 16 independent accumulators of
// v_mfma_f32_32x32x16_bf16 (all 256 accumulation registers, as a GEMM tile) and
// no memory traffic at all.  The operands are pseudo-random values (data 1: unit
// scale; data 2: unit scale against a scale of 0.02, as activations meet
// weights in the layer) or zeros (data 0): the clock the matrix cores sustain
// depends on how many bits toggle.  out[2*wg] = shader clocks, out[2*wg+1] = ticks of the
// constant 100 MHz clock spent in the loop by the workgroup's first wave.
__global__ __launch_bounds__(256) void mfma_loop_kernel(int iters, int data, unsigned long long *out,
                                                        float *sink) {
  yf32x16 acc[16];
#pragma unroll
  for (int i = 0; i < 16; i++)
#pragma unroll
    for (int q = 0; q < 16; q++) acc[i][q] = 0.f;
  ybf16x8 a[2], b[2];
  uint32_t s = 0x9e3779b9u * (blockIdx.x * 256u + threadIdx.x + 1u);
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int j = 0; j < 8; j++) {
      float u = 0.f, v = 0.f;  // sums of four uniform variates on [-1, 1): bell-shaped, variance 4/3
#pragma unroll
      for (int r = 0; r < 4; r++) {
        s = s * 1664525u + 1013904223u;
        u += (float)(s >> 8) * (1.0f / 8388608.0f) - 1.0f;
        s = s * 1664525u + 1013904223u;
        v += (float)(s >> 8) * (1.0f / 8388608.0f) - 1.0f;
      }
      // data 1: both operands of unit scale; data 2: as the layer's GEMMs see them,
      // activations of unit scale against weights of scale 0.02; data 0: zeros
      a[h][j] = (__bf16)(data ? 0.866f * u : 0.f);
      b[h][j] = (__bf16)(data == 1 ? 0.866f * v : (data == 2 ? 0.0173f * v : 0.f));
    }
  const unsigned long long c0 = clock64(), t0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 16; i++)
      acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i & 1], b[(i >> 1) & 1], acc[i], 0, 0, 0);
  }
  const unsigned long long c1 = clock64(), t1 = wall_clock64();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < 16; i++) r += acc[i][0];
  if (r == 123.456f) sink[0] = r;  // keeps the loop alive
  if (threadIdx.x == 0) {
    out[2 * blockIdx.x] = c1 - c0;
    out[2 * blockIdx.x + 1] = t1 - t0;
  }
}

// dst = src: every wave takes blocks of 16 KB in turn, 16 loads of 1 KB in flight, then 16 stores
__global__ __launch_bounds__(256) void copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                   size_t n) {
  const int lane = threadIdx.x & 63;
  const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const size_t n_waves = (size_t)gridDim.x * 4;
  const size_t n_blocks = n / 1024;  // 16 KB = 1024 uint4
  for (size_t b = wave; b < n_blocks; b += n_waves) {
    const uint4 *p = src + b * 1024 + lane;
    uint4 *q = dst + b * 1024 + lane;
    uint4 v[16];
#pragma unroll
    for (int j = 0; j < 16; j++) v[j] = p[j * 64];
#pragma unroll
    for (int j = 0; j < 16; j++) q[j * 64] = v[j];
  }
}

// reads src once: every wave takes blocks of 16 KB in turn, 16 loads of 1 KB in
// flight each, and keeps one word per workgroup
__global__ __launch_bounds__(256) void read_kernel(const uint4 *__restrict__ src, uint32_t *__restrict__ sink,
                                                   size_t n) {
  uint32_t x = 0;
  const int lane = threadIdx.x & 63;
  const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const size_t n_waves = (size_t)gridDim.x * 4;
  const size_t n_blocks = n / 1024;  // 16 KB = 1024 uint4
  for (size_t b = wave; b < n_blocks; b += n_waves) {
    const uint4 *p = src + b * 1024 + lane;
    uint4 v[16];
#pragma unroll
    for (int j = 0; j < 16; j++) v[j] = p[j * 64];
#pragma unroll
    for (int j = 0; j < 16; j++) x ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  if (x == 0x12345678u) sink[blockIdx.x] = x;
}

#define Y_TRY(call)                                                                                  \
  do {                                                                                               \
    hipError_t e_ = (call);                                                                          \
    if (e_ != hipSuccess) {                                                                          \
      rc = set_error(MOE_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__,  \
                     __LINE__);                                                                      \
      goto done;                                                                                     \
    }                                                                                                \
  } while (0)

}  // namespace
}  // namespace moe

using namespace moe;

extern "C" int moe_yardstick_mfma(int n_workgroups, int iters, int data, double *tflops,
                                  double *shader_ghz) {
  if (n_workgroups < 1 || n_workgroups > 4096 || iters < 1 || iters > (1 << 22) || !tflops)
    return set_error(MOE_ERR_BAD_ARG, "moe_yardstick_mfma: bad arguments");
  int rc = MOE_OK;
  unsigned long long *out = nullptr;
  float *sink = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  unsigned long long *host = new unsigned long long[2 * (size_t)n_workgroups];
  float ms = 0.f;
  Y_TRY(hipMalloc(reinterpret_cast<void **>(&out), sizeof(unsigned long long) * 2 * n_workgroups));
  Y_TRY(hipMalloc(reinterpret_cast<void **>(&sink), sizeof(float)));
  Y_TRY(hipEventCreate(&e0));
  Y_TRY(hipEventCreate(&e1));
  // an untimed launch of the same length first: the clocks settle under load
  mfma_loop_kernel<<<n_workgroups, 256>>>(iters, data, out, sink);
  Y_TRY(hipGetLastError());
  Y_TRY(hipEventRecord(e0, nullptr));
  mfma_loop_kernel<<<n_workgroups, 256>>>(iters, data, out, sink);
  Y_TRY(hipGetLastError());
  Y_TRY(hipEventRecord(e1, nullptr));
  Y_TRY(hipEventSynchronize(e1));
  Y_TRY(hipEventElapsedTime(&ms, e0, e1));
  Y_TRY(hipMemcpy(host, out, sizeof(unsigned long long) * 2 * n_workgroups, hipMemcpyDeviceToHost));
  {
    double clk = 0, ticks = 0;
    for (int i = 0; i < n_workgroups; i++) {
      clk += (double)host[2 * i];
      ticks += (double)host[2 * i + 1];
    }
    const double flop = (double)n_workgroups * 4 * iters * 16 * 2.0 * 32 * 32 * 16;
    *tflops = flop / (ms * 1e-3) / 1e12;
    if (shader_ghz) *shader_ghz = ticks > 0 ? clk / (ticks * 10.0) : 0.0;  // 100 MHz ticks -> ns
  }
done:
  delete[] host;
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(out);
  (void)hipFree(sink);
  return rc;
}

extern "C" int moe_yardstick_hbm(size_t bytes, int iters, double *copy_gbs, double *read_gbs) {
  if (bytes < (1u << 20) || (bytes & 16383) || iters < 1 || iters > 1000 || !copy_gbs || !read_gbs)
    return set_error(MOE_ERR_BAD_ARG, "moe_yardstick_hbm: bad arguments");
  int rc = MOE_OK;
  uint4 *src = nullptr, *dst = nullptr;
  uint32_t *sink = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr, e2 = nullptr;
  const size_t n = bytes / 16;
  const int grid = 256 * 8;
  float ms_copy = 0.f, ms_read = 0.f;
  Y_TRY(hipMalloc(reinterpret_cast<void **>(&src), bytes));
  Y_TRY(hipMalloc(reinterpret_cast<void **>(&dst), bytes));
  Y_TRY(hipMalloc(reinterpret_cast<void **>(&sink), sizeof(uint32_t) * grid));
  Y_TRY(hipMemset(src, 0x5a, bytes));
  Y_TRY(hipMemset(dst, 0, bytes));
  Y_TRY(hipEventCreate(&e0));
  Y_TRY(hipEventCreate(&e1));
  Y_TRY(hipEventCreate(&e2));
  copy_kernel<<<grid, 256>>>(src, dst, n);
  read_kernel<<<grid, 256>>>(src, sink, n);
  Y_TRY(hipGetLastError());
  Y_TRY(hipEventRecord(e0, nullptr));
  for (int i = 0; i < iters; i++) copy_kernel<<<grid, 256>>>(src, dst, n);
  Y_TRY(hipEventRecord(e1, nullptr));
  for (int i = 0; i < iters; i++) read_kernel<<<grid, 256>>>(src, sink, n);
  Y_TRY(hipGetLastError());
  Y_TRY(hipEventRecord(e2, nullptr));
  Y_TRY(hipEventSynchronize(e2));
  Y_TRY(hipEventElapsedTime(&ms_copy, e0, e1));
  Y_TRY(hipEventElapsedTime(&ms_read, e1, e2));
  *copy_gbs = 2.0 * (double)bytes * iters / (ms_copy * 1e-3) / 1e9;  // bytes read + bytes written
  *read_gbs = (double)bytes * iters / (ms_read * 1e-3) / 1e9;
done:
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (e2) (void)hipEventDestroy(e2);
  (void)hipFree(src);
  (void)hipFree(dst);
  (void)hipFree(sink);
  return rc;
}
