// Stand-alone measurement tool (not part of the library):
//   ingest_probe mfma     sustained rate of v_mfma_f32_32x32x16_bf16 from registers
//                         alone, and the shader clock it runs at, for 64 / 128 /
//                         256 busy CUs
//   ingest_probe stream   per-CU streaming rate L2/MALL/HBM -> LDS (DMA) and -> VGPR
//   ingest_probe copy N   one plain copy kernel of N MiB, for calibrating the
//                         FETCH_SIZE / WRITE_SIZE counters of rocprofv3 --pmc
// The figures bound what a GEMM tile may read per clock and are quoted in the
// design notes; they are hardware properties, nothing here is tuned.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

#define CK(x)                                                                      \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);        \
      exit(1);                                                                     \
    }                                                                              \
  } while (0)

__device__ __forceinline__ void dma16(const uint4 *g, uint4 *lds) {
  const uint32_t m = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m), "v"(g)
               : "memory");
}

// Every wave keeps 16 loads of 1 KB in flight; a workgroup of NW waves walks
// through `span_chunks` 16-byte chunks with a stride that spreads workgroups.
template <int NW, bool TO_LDS>
__global__ __launch_bounds__(NW * 64) void stream_kernel(const uint4 *src, size_t span_chunks,
                                                        int iters, uint4 *sink) {
  __shared__ uint4 lds[NW * 16 * 64];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const size_t base = ((size_t)blockIdx.x * 977 * NW + w) * 64;
  uint4 acc = make_uint4(0, 0, 0, 0);
  for (int it = 0; it < iters; it++) {
    if (TO_LDS) {
#pragma unroll
      for (int j = 0; j < 16; j++) {
        const size_t idx = (base + (size_t)(it * 16 + j) * NW * 64) % span_chunks;
        dma16(src + idx + lane, lds + (w * 16 + j) * 64);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
      uint4 v[16];
#pragma unroll
      for (int j = 0; j < 16; j++) {
        const size_t idx = (base + (size_t)(it * 16 + j) * NW * 64) % span_chunks;
        v[j] = src[idx + lane];
      }
#pragma unroll
      for (int j = 0; j < 16; j++) {
        acc.x ^= v[j].x; acc.y ^= v[j].y; acc.z ^= v[j].z; acc.w ^= v[j].w;
      }
    }
  }
  if (TO_LDS) {
    __syncthreads();
    acc = lds[threadIdx.x];
  }
  if (acc.x == 0x12345678u) sink[threadIdx.x] = acc;  // keeps the loads alive
}

template <int NW, bool TO_LDS>
static void run_stream(const char *name, const uint4 *src, size_t span_bytes, uint4 *sink, int grid) {
  const int iters = 64;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  stream_kernel<NW, TO_LDS><<<grid, NW * 64>>>(src, span_bytes / 16, iters, sink);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  for (int r = 0; r < 5; r++)
    stream_kernel<NW, TO_LDS><<<grid, NW * 64>>>(src, span_bytes / 16, iters, sink);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  const double bytes = 5.0 * grid * NW * 64 * 16.0 * 16 * iters;
  printf("%-26s span %7.1f MB  workgroups %4d x %d waves : %6.2f TB/s  %5.1f GB/s per workgroup\n",
         name, span_bytes / 1e6, grid, NW, bytes / ms / 1e9, bytes / ms / 1e6 / grid);
}

__global__ void copy_kernel(const uint4 *src, uint4 *dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// 4 waves per workgroup, one per SIMD; 16 independent accumulators per wave, no
// memory traffic.  out[2*wg] = shader clocks (s_memtime), out[2*wg+1] = 100 MHz
// ticks (s_memrealtime) spent in the loop.
__global__ __launch_bounds__(256) void mfma_kernel(int iters, unsigned long long *out, float *sink) {
  f32x16_t acc[16];
#pragma unroll
  for (int i = 0; i < 16; i++)
#pragma unroll
    for (int q = 0; q < 16; q++) acc[i][q] = 0.f;
  bf16x8_t a, b;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    a[j] = (__bf16)(0.001f * (float)(threadIdx.x + j));
    b[j] = (__bf16)(0.002f * (float)(threadIdx.x ^ j));
  }
  const unsigned long long c0 = clock64(), t0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
  }
  const unsigned long long c1 = clock64(), t1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; i++) s += acc[i][0];
  if (s == 123.456f) sink[0] = s;
  if (threadIdx.x == 0) {
    out[2 * blockIdx.x] = c1 - c0;
    out[2 * blockIdx.x + 1] = t1 - t0;
  }
}

static void run_mfma(int grid) {
  const int iters = 20000;  // x 16 MFMAs of 32 clocks: about 5 ms
  unsigned long long *out, host[2 * 256];
  float *sink;
  CK(hipMalloc(&out, sizeof host));
  CK(hipMalloc(&sink, 4));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  mfma_kernel<<<grid, 256>>>(1000, out, sink);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  mfma_kernel<<<grid, 256>>>(iters, out, sink);
  CK(hipEventRecord(e1));
  CK(hipDeviceSynchronize());
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  CK(hipMemcpy(host, out, sizeof(unsigned long long) * 2 * grid, hipMemcpyDeviceToHost));
  double clk = 0, ticks = 0;
  for (int i = 0; i < grid; i++) { clk += (double)host[2 * i]; ticks += (double)host[2 * i + 1]; }
  const double flop = (double)grid * 4 * iters * 16 * 2.0 * 32 * 32 * 16;
  printf("%3d workgroups (one per CU): %7.1f TFLOP/s, shader clock %.2f GHz, %.1f clocks per MFMA per SIMD\n",
         grid, flop / (ms * 1e-3) / 1e12, clk / (ticks * 10.0), clk / grid / ((double)iters * 16));
  CK(hipFree(out));
  CK(hipFree(sink));
}

int main(int argc, char **argv) {
  if (argc >= 2 && !strcmp(argv[1], "mfma")) {
    for (int grid : {64, 128, 256}) run_mfma(grid);
    return 0;
  }
  if (argc >= 3 && !strcmp(argv[1], "copy")) {
    const size_t bytes = (size_t)atol(argv[2]) << 20;
    uint4 *a, *b;
    CK(hipMalloc(&a, bytes));
    CK(hipMalloc(&b, bytes));
    CK(hipMemset(a, 1, bytes));
    CK(hipDeviceSynchronize());
    copy_kernel<<<4096, 256>>>(a, b, bytes / 16);
    CK(hipDeviceSynchronize());
    printf("copy_kernel moved %zu MiB: reads %zu KiB, writes %zu KiB\n", bytes >> 20, bytes >> 10,
           bytes >> 10);
    return 0;
  }
  const size_t big = (size_t)2 << 30;
  uint4 *src, *sink;
  CK(hipMalloc(&src, big));
  CK(hipMalloc(&sink, 1 << 20));
  CK(hipMemset(src, 1, big));
  for (size_t span : {(size_t)8 << 20, (size_t)128 << 20, big}) {
    run_stream<4, true>("L2->LDS  (DMA x4)", src, span, sink, 256);
    run_stream<8, true>("L2->LDS  (DMA x4)", src, span, sink, 256);
    run_stream<8, true>("L2->LDS  (DMA x4)", src, span, sink, 512);
    run_stream<4, false>("L2->VGPR (load x4)", src, span, sink, 256);
    run_stream<8, false>("L2->VGPR (load x4)", src, span, sink, 256);
  }
  for (int grid : {8, 64, 128})
    run_stream<8, true>("L2->LDS, few workgroups", src, (size_t)8 << 20, sink, grid);
  return 0;
}
