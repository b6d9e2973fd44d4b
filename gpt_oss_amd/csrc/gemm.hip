// Grouped expert GEMMs on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16,
// fp32 accumulate).  Replaces mlp1_kernel / mlp1_120b_kernel
// (matmul/matmul.cpp:1023-1465) with the clamped SwiGLU in the epilogue
// (utility/utility.cpp:1108-1125; formula of run.cpp:709-726) and
// mlp2_kernel_noatomic / mlp2_120b_kernel (matmul/matmul.cpp:1470-1914).
//
// Data layout.  Both operands arrive as ready-made MFMA fragments of 1 KB
// (64 lanes x 8 bf16, see pack.hip and gather_rows_kernel), ordered
// [row block of 32][k block of 16], so every global load is a contiguous
// 16 bytes per lane and lands in LDS in register order: LDS reads are
// lane-linear ds_read_b128, free of bank conflicts by construction.
//
// Tiling.  A workgroup of 4 waves (2 x 2) owns a tile of (2*RB*32) rows x
// (2*NBW*32) columns of one expert; a wave keeps RB x NBW accumulators of
// 32x32.  RB follows the expert's row count (ExpertInfo::rb) so that ragged
// segments pad to at most 63 rows.  The reduction runs in steps of KPS k
// blocks through a 2-stage LDS ring that global_load_lds (buffer-less DMA
// into LDS) fills one step ahead of the MFMAs.
//
// Tile order.  Workgroup ids are dealt round-robin to the 8 XCDs, each with
// its own L2.  Logical tile ids are laid out (expert, column tile, row tile)
// with the row tile fastest, and XCD x takes the x-th contiguous eighth of
// them: the tiles an XCD runs at one time share the expert's rows and a few
// column slabs of its weights, so each weight byte leaves HBM once.
#include "moe_internal.h"

namespace moe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint16_t f32_to_bf16_rne_dev(float f) {
  uint32_t u = __float_as_uint(f);
  u += 0x7fffu + ((u >> 16) & 1u);  // finite inputs only
  return (uint16_t)(u >> 16);
}

// run.cpp:709-726: gate clamped from above, up clamped on both sides.
__device__ __forceinline__ float swiglu(float g, float u, float limit) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  const float s = __builtin_amdgcn_rcpf(1.0f + __expf(-kAlpha * g));
  return g * s * (u + 1.0f);
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding).
#define WAIT_VMCNT(n) \
  __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | (0x7 << 4) | (0xf << 8))

struct TileCoord {
  int e;      // expert
  int rb0;    // first row block (32 rows) of the tile in the padded row space
  int nt;     // column tile
  int rows0;  // first row of the tile relative to the expert's segment
};

// Maps the workgroup id to a tile (see "Tile order" above).  Returns false for
// the surplus workgroups of the upper-bound grid.
__device__ __forceinline__ bool locate_tile(const ExpertInfo *__restrict__ info,
                                            const int *__restrict__ totals, int E, int n_ct,
                                            TileCoord &tc, int &rb) {
  const int total = totals[0] * n_ct;
  const int per_xcd = (total + 7) >> 3;
  const int bid = blockIdx.x;
  const int idx = bid >> 3;
  if (idx >= per_xcd) return false;
  const int L = (bid & 7) * per_xcd + idx;
  if (L >= total) return false;
  // largest e with tile_base[e] * n_ct <= L and n_mt[e] > 0
  int lo = 0, hi = E - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (info[mid].tile_base * n_ct <= L) lo = mid; else hi = mid - 1;
  }
  // An expert without rows shares tile_base with its successor, so the search
  // passes over it; a trailing run of empty experts has tile_base == totals[0]
  // and cannot be reached because L < total.
  const int e = lo;
  const ExpertInfo inf = info[e];
  const int rem = L - inf.tile_base * n_ct;
  const int mt = rem % inf.n_mt;
  tc.e = e;
  tc.nt = rem / inf.n_mt;
  rb = inf.rb;
  tc.rows0 = mt * 2 * rb * kRowBlock;
  tc.rb0 = (inf.row0 + tc.rows0) / kRowBlock;
  return true;
}

template <int RB, int NBW, int KPS, bool GATE_UP>
__device__ __forceinline__ void gemm_tile(const uint4 *__restrict__ a_frag,  // [rb][KB][64]
                                          const uint4 *__restrict__ b_frag,  // expert: [nb][KB][64]
                                          int KB, int rb0, int nb0, int nb_valid,
                                          const float *__restrict__ bias_a,  // gate / down bias (expert)
                                          const float *__restrict__ bias_b,  // up bias (expert)
                                          void *__restrict__ outp, int out_ld, float limit,
                                          uint4 *lds) {
  constexpr int A_CH = 2 * RB * KPS;   // 1 KB chunks of A per stage
  constexpr int B_CH = 2 * NBW * KPS;  // 1 KB chunks of B per stage
  constexpr int STAGE = (A_CH + B_CH) * 64;  // in uint4
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;

  f32x16 acc[RB][NBW];
#pragma unroll
  for (int i = 0; i < RB; i++)
#pragma unroll
    for (int j = 0; j < NBW; j++)
#pragma unroll
      for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;

  // Chunk c of a stage (c = pass*4 + wave) covers row block c / KPS, k block c % KPS.
  auto issue = [&](int stage, int ks) {
    uint4 *sa = lds + stage * STAGE;
    uint4 *sb = sa + A_CH * 64;
#pragma unroll
    for (int c0 = 0; c0 < A_CH; c0 += 4) {
      const int c = c0 + w;
      if (A_CH % 4 == 0 || c < A_CH) {
        const uint4 *g = a_frag + ((size_t)(rb0 + c / KPS) * KB + ks * KPS + c % KPS) * 64 + lane;
        __builtin_amdgcn_global_load_lds(g, sa + c * 64, 16, 0, 0);
      }
    }
#pragma unroll
    for (int c0 = 0; c0 < B_CH; c0 += 4) {
      const int c = c0 + w;
      if (B_CH % 4 == 0 || c < B_CH) {
        // Column blocks past the end of the matrix (last column tile only) re-load
        // the last valid block instead of branching; their products are never stored.
        const int nb = min(c / KPS, nb_valid - 1);
        const uint4 *g = b_frag + ((size_t)(nb0 + nb) * KB + ks * KPS + c % KPS) * 64 + lane;
        __builtin_amdgcn_global_load_lds(g, sb + c * 64, 16, 0, 0);
      }
    }
  };

  const int n_steps = KB / KPS;
  issue(0, 0);
  for (int ks = 0; ks < n_steps; ks++) {
    WAIT_VMCNT(0);
    __syncthreads();  // step ks is in LDS; every wave is done reading step ks-1
    if (ks + 1 < n_steps) issue((ks + 1) & 1, ks + 1);
    const uint4 *sa = lds + (ks & 1) * STAGE;
    const uint4 *sb = sa + A_CH * 64;
#pragma unroll
    for (int kk = 0; kk < KPS; kk++) {
      bf16x8 a[RB], b[NBW];
#pragma unroll
      for (int i = 0; i < RB; i++) {
        const uint4 v = sa[((wm * RB + i) * KPS + kk) * 64 + lane];
        a[i] = __builtin_bit_cast(bf16x8, v);
      }
#pragma unroll
      for (int j = 0; j < NBW; j++) {
        const uint4 v = sb[((wn * NBW + j) * KPS + kk) * 64 + lane];
        b[j] = __builtin_bit_cast(bf16x8, v);
      }
#pragma unroll
      for (int i = 0; i < RB; i++)
#pragma unroll
        for (int j = 0; j < NBW; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }

  // Epilogue.  Accumulator register q of lane l is row 8*(q/4) + 4*(l/32) + q%4,
  // column l % 32 of its 32x32 block.
  const int n = lane & 31;
  const int rsub = 4 * (lane >> 5);
  if (GATE_UP) {
    // Column blocks come in (gate, up) pairs; pair P yields activation columns
    // 32*P .. 32*P+31.  The result is written as bf16 in the fragment order the
    // down GEMM reads as its A operand: k block = col / 16, lane = ((col%16)/8)*32
    // + row%32, element col % 8.
    uint16_t *act = reinterpret_cast<uint16_t *>(outp);
    const int kb2_total = out_ld / kFragK;
#pragma unroll
    for (int j = 0; j < NBW; j += 2) {
      if (wn * NBW + j >= nb_valid) continue;
      const int P = (nb0 + wn * NBW + j) >> 1;
      const int col = kRowBlock * P + n;
      const float bg = bias_a[col];
      const float bu = bias_b[col];
      const int kb2 = col / kFragK;
      const int lane_hi = ((col % kFragK) / 8) * 32;
#pragma unroll
      for (int i = 0; i < RB; i++) {
        const size_t frag = (size_t)(rb0 + wm * RB + i) * kb2_total + kb2;
#pragma unroll
        for (int q = 0; q < 16; q++) {
          const int r = 8 * (q >> 2) + rsub + (q & 3);
          const float v = swiglu(acc[i][j][q] + bg, acc[i][j + 1][q] + bu, limit);
          act[(frag * 64 + lane_hi + r) * 8 + (col & 7)] = f32_to_bf16_rne_dev(v);
        }
      }
    }
  } else {
    float *y = reinterpret_cast<float *>(outp);
#pragma unroll
    for (int j = 0; j < NBW; j++) {
      if (wn * NBW + j >= nb_valid) continue;
      const int col = kRowBlock * (nb0 + wn * NBW + j) + n;
      const float bb = bias_a[col];
#pragma unroll
      for (int i = 0; i < RB; i++) {
        const size_t row0 = (size_t)(rb0 + wm * RB + i) * kRowBlock;
#pragma unroll
        for (int q = 0; q < 16; q++) {
          const int r = 8 * (q >> 2) + rsub + (q & 3);
          y[(row0 + r) * out_ld + col] = acc[i][j][q] + bb;
        }
      }
    }
  }
}

template <int NBW, int KPS, bool GATE_UP>
__global__ __launch_bounds__(256) void grouped_gemm_kernel(
    const uint4 *__restrict__ a_frag, const uint4 *__restrict__ w_frag,
    const float *__restrict__ bias_a, const float *__restrict__ bias_b,
    const ExpertInfo *__restrict__ info, const int *__restrict__ totals, void *__restrict__ outp,
    int K, int N, int E, float limit) {
  extern __shared__ uint4 lds[];
  const int KB = K / kFragK;
  const int nb_total = (GATE_UP ? 2 * N : N) / kRowBlock;  // weight row blocks per expert
  const int n_ct = (nb_total + 2 * NBW - 1) / (2 * NBW);
  TileCoord tc;
  int rb;
  if (!locate_tile(info, totals, E, n_ct, tc, rb)) return;
  const int nb0 = tc.nt * 2 * NBW;
  const int nb_valid = min(2 * NBW, nb_total - nb0);
  const uint4 *b_frag = w_frag + (size_t)tc.e * nb_total * KB * 64;
  const float *ba = bias_a + (size_t)tc.e * N;
  const float *bb = GATE_UP ? bias_b + (size_t)tc.e * N : nullptr;
  switch (rb) {
    case 1: gemm_tile<1, NBW, KPS, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, lds); break;
    case 2: gemm_tile<2, NBW, KPS, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, lds); break;
    case 3: gemm_tile<3, NBW, KPS, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, lds); break;
    default: gemm_tile<4, NBW, KPS, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, lds); break;
  }
}

constexpr int kKps = 4;  // k blocks (of 16) per pipeline step

template <int NBW>
constexpr size_t lds_bytes() {
  return (size_t)2 * (2 * 4 + 2 * NBW) * kKps * kFragBytes;
}

hipError_t launch_gate_up(const uint16_t *xg, const uint16_t *w1, const float *b1g, const float *b1u,
                          const DispatchBuffers &d, uint16_t *act, int H, int IM, int E, float limit,
                          int mt_cap, hipStream_t s) {
  constexpr int NBW = kNbwGateUp;
  const int nb_total = 2 * IM / kRowBlock;
  const int n_ct = (nb_total + 2 * NBW - 1) / (2 * NBW);
  const int grid = ((mt_cap * n_ct + 7) / 8) * 8;
  auto kern = grouped_gemm_kernel<NBW, kKps, true>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes<NBW>());
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  kern<<<grid, 256, lds_bytes<NBW>(), s>>>(reinterpret_cast<const uint4 *>(xg),
                                          reinterpret_cast<const uint4 *>(w1), b1g, b1u, d.info,
                                          d.totals, act, H, IM, E, limit);
  return hipGetLastError();
}

hipError_t launch_down(const uint16_t *act, const uint16_t *w2, const float *b2,
                       const DispatchBuffers &d, float *y, int H, int IM, int E, int mt_cap,
                       hipStream_t s) {
  constexpr int NBW = kNbwDown;
  const int nb_total = H / kRowBlock;
  const int n_ct = (nb_total + 2 * NBW - 1) / (2 * NBW);
  const int grid = ((mt_cap * n_ct + 7) / 8) * 8;
  auto kern = grouped_gemm_kernel<NBW, kKps, false>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes<NBW>());
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  kern<<<grid, 256, lds_bytes<NBW>(), s>>>(reinterpret_cast<const uint4 *>(act),
                                          reinterpret_cast<const uint4 *>(w2), b2, nullptr, d.info,
                                          d.totals, y, IM, H, E, 0.f);
  return hipGetLastError();
}

}  // namespace moe
