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
// Tiling.  A workgroup of WM x WN waves owns a tile of (WM*RB*32) rows x
// (WN*NBW*32) columns of one expert; a wave keeps RB x NBW accumulators of
// 32x32.  RB follows the expert's row count (ExpertInfo::rb) so that ragged
// segments pad to at most 63 rows.  The reduction runs in steps of KPS k
// blocks through a 4-stage LDS ring that global_load_lds (DMA into LDS, no
// staging registers) keeps three steps ahead of the MFMAs.
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

// LDS ring: one __shared__ array per stage, so that the compiler can tell a
// read of one stage from the DMA that fills another and does not serialise them.
template <int NST>
struct StageRing {
  uint4 *p[NST];
};

// Workgroup barrier that orders LDS traffic only.  A __syncthreads (or a
// workgroup fence) would also drain the vector-memory counter and with it the
// DMA of the steps still in flight; those are covered by the explicit vmcnt
// waits of the pipeline.  The memory clobber keeps the compiler from moving
// LDS accesses across the barrier.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 16 bytes per lane from global memory straight into LDS at base + 16*lane
// (global_load_lds_dwordx4; M0 carries the wave-uniform LDS base).  Issued as
// inline assembly on purpose: the compiler then does not pair the LDS write with
// later ds_reads of OTHER stages and drain the whole queue before them; the
// pipeline's own vmcnt waits order the read of a stage after its fill.
__device__ __forceinline__ void dma_to_lds_16(const uint4 *g, uint4 *lds_wave_base) {
  const uint32_t m = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds_wave_base;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(m), "v"(g)
               : "memory");
}

// Shape of one workgroup: WM x WN waves, each owning RB x NBW accumulators of
// 32x32; the tile is (WM*RB*32) rows x (WN*NBW*32) columns.  KPS k blocks per
// pipeline step, NST LDS stages.
template <int WM_, int WN_, int NBW_, int KPS_, int NST_>
struct GemmCfg {
  static constexpr int WM = WM_, WN = WN_, NBW = NBW_, KPS = KPS_, NST = NST_;
  static constexpr int NW = WM * WN;              // waves
  static constexpr int THREADS = NW * 64;
  static constexpr int RB_MAX = kTileRows / (WM * kRowBlock);
  static constexpr int TILE_NB = WN * NBW;        // column blocks per tile
  static constexpr int B_OFF = WM * RB_MAX * KPS * 64;             // B follows the tallest A, in uint4
  static constexpr int STAGE = (WM * RB_MAX + WN * NBW) * KPS * 64;  // uint4 per stage
};

template <int RB, typename C, bool GATE_UP>
__device__ __forceinline__ void gemm_tile(const uint4 *__restrict__ a_frag,  // [rb][KB][64]
                                          const uint4 *__restrict__ b_frag,  // expert: [nb][KB][64]
                                          int KB, int rb0, int nb0, int nb_valid,
                                          const float *__restrict__ bias_a,  // gate / down bias (expert)
                                          const float *__restrict__ bias_b,  // up bias (expert)
                                          void *__restrict__ outp, int out_ld, float limit,
                                          const StageRing<C::NST> &ring) {
  constexpr int WN = C::WN, NBW = C::NBW, KPS = C::KPS, NST = C::NST, NW = C::NW;
  static_assert(KPS == 2, "the step is software-pipelined as two k blocks");
  constexpr int A_CH = C::WM * RB * KPS;  // 1 KB chunks of A per stage
  constexpr int B_CH = WN * NBW * KPS;    // 1 KB chunks of B per stage
  static_assert(A_CH % NW == 0 && B_CH % NW == 0, "every wave issues the same number of loads");
  constexpr int LPS = (A_CH + B_CH) / NW;  // DMA loads per wave per step
  constexpr int NF = RB + NBW;             // fragments a wave reads per k block
  constexpr int NM = RB * NBW;             // MFMAs per k block
  constexpr int SIDE1 = (NF + NM - 1) / NM;        // side items per MFMA, first k block
  constexpr int SIDE2 = (LPS + NF + NM - 1) / NM;  // second k block
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w / WN, wn = w % WN;

  f32x16 acc[RB][NBW];
#pragma unroll
  for (int i = 0; i < RB; i++)
#pragma unroll
    for (int j = 0; j < NBW; j++)
#pragma unroll
      for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;

  // DMA chunk c of a stage (c = pass*NW + wave) covers row block c / KPS, k block
  // c % KPS.  Load m (0 <= m < LPS) of this wave: first its A chunks, then its B chunks.
  const uint4 *a_src = a_frag + (size_t)rb0 * KB * 64 + lane;
  const uint4 *b_src = b_frag + (size_t)nb0 * KB * 64 + lane;
  auto issue_one = [&](uint4 *st, int ks, int m) {
    if (m < A_CH / NW) {
      const int c = m * NW + w;
      const uint4 *g = a_src + ((size_t)(c / KPS) * KB + ks * KPS + c % KPS) * 64;
      dma_to_lds_16(g, st + c * 64);
    } else {
      const int c = (m - A_CH / NW) * NW + w;
      // Column blocks past the end of the matrix (last column tile only) re-load
      // the last valid block instead of branching; their products are never stored.
      const int nb = min(c / KPS, nb_valid - 1);
      const uint4 *g = b_src + ((size_t)nb * KB + ks * KPS + c % KPS) * 64;
      dma_to_lds_16(g, st + C::B_OFF + c * 64);
    }
  };
  auto issue = [&](uint4 *st, int ks) {
#pragma unroll
    for (int m = 0; m < LPS; m++) issue_one(st, ks, m);
  };

  // Two register sets of fragments: while the MFMAs of one k block run, the
  // fragments of the next are read from LDS.
  bf16x8 fa[2][RB], fb[2][NBW];
  auto read_frag = [&](const uint4 *st, int kk, int buf, int f) {
    if (f < RB) {
      fa[buf][f] = __builtin_bit_cast(bf16x8, st[((wm * RB + f) * KPS + kk) * 64 + lane]);
    } else {
      fb[buf][f - RB] =
          __builtin_bit_cast(bf16x8, st[C::B_OFF + ((wn * NBW + f - RB) * KPS + kk) * 64 + lane]);
    }
  };

  const int n_steps = KB / KPS;
#pragma unroll
  for (int s = 0; s < NST - 1; s++)
    if (s < n_steps) issue(ring.p[s], s);
  if (n_steps - 1 >= NST - 2) {
    WAIT_VMCNT(LPS * (NST - 2));
  } else {
    WAIT_VMCNT(0);
  }
  lds_barrier();
  if (NST - 1 < n_steps) issue(ring.p[NST - 1], NST - 1);
#pragma unroll
  for (int f = 0; f < NF; f++) read_frag(ring.p[0], 0, 0, f);

  // Step ks: [read k block 1 | MFMAs of k block 0] [wait for step ks+1, barrier]
  // [refill the stage just drained with step ks+NST, read k block 0 of step ks+1 |
  // MFMAs of k block 1].  The side work is spread one item per MFMA so that it
  // issues in the shadow of the matrix pipe.
  for (int ks0 = 0; ks0 < n_steps; ks0 += NST) {
#pragma unroll
    for (int u = 0; u < NST; u++) {
      const int ks = ks0 + u;
      if (ks < n_steps) {
      const uint4 *cur = ring.p[u];
#pragma unroll
      for (int m = 0; m < NM; m++) {
#pragma unroll
        for (int t = m * SIDE1; t < (m + 1) * SIDE1; t++)
          if (t < NF) read_frag(cur, 1, 1, t);
        acc[m / NBW][m % NBW] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            fa[0][m / NBW], fb[0][m % NBW], acc[m / NBW][m % NBW], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      const bool more = ks + 1 < n_steps;
      const bool refill = ks + NST < n_steps;
      if (more) {
        if (ks + NST - 1 < n_steps) {
          WAIT_VMCNT(LPS * (NST - 2));  // all but the NST-2 newest steps have landed
        } else {
          WAIT_VMCNT(0);
        }
        lds_barrier();  // step ks+1 is complete in LDS; every wave is done with stage u
      }
      const uint4 *nxt = ring.p[(u + 1) % NST];
#pragma unroll
      for (int m = 0; m < NM; m++) {
#pragma unroll
        for (int t = m * SIDE2; t < (m + 1) * SIDE2; t++) {
          if (t < LPS) {
            if (refill) issue_one(ring.p[u], ks + NST, t);
          } else if (t < LPS + NF) {
            if (more) read_frag(nxt, 0, 0, t - LPS);
          }
        }
        acc[m / NBW][m % NBW] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            fa[1][m / NBW], fb[1][m % NBW], acc[m / NBW][m % NBW], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      }
    }
  }

  // Epilogue.  Accumulator register q of lane l is row 8*(q/4) + 4*(l/32) + q%4,
  // column l % 32 of its 32x32 block.  Results are re-ordered through LDS (the
  // pipeline stages are idle now; each wave takes a private piece) so that they
  // leave as 16 bytes per lane, 1 KB contiguous per wave store.
  lds_barrier();  // every wave has finished reading the stages
  static_assert(NW <= NST, "one stage per wave serves as its epilogue buffer");
  uint4 *ebuf = ring.p[w];
  const int n = lane & 31;
  const int rsub = 4 * (lane >> 5);
  if (GATE_UP) {
    // Column blocks come in (gate, up) pairs (see pack_weight_kernel): blocks 2P
    // and 2P+1 of the product hold gate_j and up_j of j = 32P .. 32P+31 in the
    // same lane and register.  The activation goes out as bf16 in the fragment
    // order the down GEMM reads as its A operand: column j is k block j/16,
    // lane ((j%16)/8)*32 + row, element j % 8.
    static_assert(NBW % 2 == 0, "gate and up blocks of a pair must sit in one wave");
    static_assert(NBW * 64 <= C::STAGE, "epilogue buffer");
    uint4 *act = reinterpret_cast<uint4 *>(outp);
    uint16_t *e16 = reinterpret_cast<uint16_t *>(ebuf);
    const int kb2_total = out_ld / kFragK;
    const int P0 = (nb0 + wn * NBW) >> 1;       // first pair of this wave
    const int pairs_valid = (nb_valid - wn * NBW) >> 1;  // may be <= 0 in the last column tile
    float bg[NBW / 2], bu[NBW / 2];
#pragma unroll
    for (int p = 0; p < NBW / 2; p++) {
      const int P = min(P0 + p, ((nb0 + nb_valid) >> 1) - 1);
      bg[p] = bias_a[kRowBlock * P + n];
      bu[p] = bias_b[kRowBlock * P + n];
    }
    // element offset of (row 0, column n of pair p) inside the wave's buffer of NBW fragments
    const int e_off = ((n >> 4) * 64 + ((n & 15) >> 3) * 32) * 8 + (n & 7);
#pragma unroll
    for (int i = 0; i < RB; i++) {
#pragma unroll
      for (int p = 0; p < NBW / 2; p++) {
        uint16_t *dst = e16 + p * 2 * 64 * 8 + e_off;
#pragma unroll
        for (int q = 0; q < 16; q++) {
          const int r = 8 * (q >> 2) + rsub + (q & 3);
          dst[r * 8] = f32_to_bf16_rne_dev(
              swiglu(acc[i][2 * p][q] + bg[p], acc[i][2 * p + 1][q] + bu[p], limit));
        }
      }
      uint4 *row_dst = act + ((size_t)(rb0 + wm * RB + i) * kb2_total + 2 * P0) * 64 + lane;
#pragma unroll
      for (int f = 0; f < NBW; f++) {
        const uint4 v = ebuf[f * 64 + lane];
        if ((f >> 1) < pairs_valid) row_dst[f * 64] = v;
      }
    }
  } else {
    constexpr int LD = NBW * 32 + 8;  // floats per buffered row; +8 keeps the two lane halves on different banks
    static_assert(32 * LD * 4 <= C::STAGE * 16, "epilogue buffer");
    float *y = reinterpret_cast<float *>(outp);
    float *ef = reinterpret_cast<float *>(ebuf);
    float bb[NBW];
#pragma unroll
    for (int j = 0; j < NBW; j++) {
      const int b = min(nb0 + wn * NBW + j, nb0 + nb_valid - 1);
      bb[j] = bias_a[kRowBlock * b + n];
    }
    const int col0 = kRowBlock * (nb0 + wn * NBW);
#pragma unroll
    for (int i = 0; i < RB; i++) {
#pragma unroll
      for (int j = 0; j < NBW; j++)
#pragma unroll
        for (int q = 0; q < 16; q++) {
          const int r = 8 * (q >> 2) + rsub + (q & 3);
          ef[r * LD + 32 * j + n] = acc[i][j][q] + bb[j];
        }
      const size_t row0 = (size_t)(rb0 + wm * RB + i) * kRowBlock;
#pragma unroll
      for (int t = 0; t < NBW * 4; t++) {
        const int idx = t * 64 + lane;
        const int r = idx / (NBW * 8);
        const int c4 = idx % (NBW * 8);
        const float4 v = *reinterpret_cast<const float4 *>(ef + r * LD + 4 * c4);
        if (wn * NBW + c4 / 8 < nb_valid)
          *reinterpret_cast<float4 *>(y + (row0 + r) * out_ld + col0 + 4 * c4) = v;
      }
    }
  }
}

template <typename C, bool GATE_UP>
__global__ __launch_bounds__(C::THREADS) void grouped_gemm_kernel(
    const uint4 *__restrict__ a_frag, const uint4 *__restrict__ w_frag,
    const float *__restrict__ bias_a, const float *__restrict__ bias_b,
    const ExpertInfo *__restrict__ info, const int *__restrict__ totals, void *__restrict__ outp,
    int K, int N, int E, float limit) {
  constexpr int NST = C::NST;
  __shared__ uint4 st0[C::STAGE];
  __shared__ uint4 st1[C::STAGE];
  __shared__ uint4 st2[NST > 2 ? C::STAGE : 1];
  __shared__ uint4 st3[NST > 3 ? C::STAGE : 1];
  StageRing<NST> ring;
  ring.p[0] = st0;
  ring.p[1] = st1;
  if constexpr (NST > 2) ring.p[2] = st2;
  if constexpr (NST > 3) ring.p[3] = st3;
  const int KB = K / kFragK;
  const int nb_total = (GATE_UP ? 2 * N : N) / kRowBlock;  // weight row blocks per expert
  const int n_ct = (nb_total + C::TILE_NB - 1) / C::TILE_NB;
  TileCoord tc;
  int rb;
  if (!locate_tile(info, totals, E, n_ct, tc, rb)) return;
  const int nb0 = tc.nt * C::TILE_NB;
  const int nb_valid = min(C::TILE_NB, nb_total - nb0);
  const uint4 *b_frag = w_frag + (size_t)tc.e * nb_total * KB * 64;
  const float *ba = bias_a + (size_t)tc.e * N;
  const float *bb = GATE_UP ? bias_b + (size_t)tc.e * N : nullptr;
  switch (rb) {
    case 1: gemm_tile<1, C, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, ring); break;
    case 2: gemm_tile<2, C, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, ring); break;
    case 3: gemm_tile<3, C, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, ring); break;
    default: gemm_tile<4, C, GATE_UP>(a_frag, b_frag, KB, tc.rb0, nb0, nb_valid, ba, bb, outp, N, limit, ring); break;
  }
}

// 4 waves (2 x 2), one per SIMD, each with 4 x 5 accumulators (320 registers).
// Tiles are 256 x 320: a CU takes in at most about 21 bytes per clock from L2,
// so the arithmetic per byte of the tile, 2*256*320 flops per (256+320)*2
// bytes for every unit of k, bounds the MFMA rate; 320 also divides both
// 2*IM = 5760 and H = 2880 at the GPT-OSS shapes, so no column tile is partial.
// 2 k blocks per step, 4 stages of 36 KB.
using CfgGateUp = GemmCfg<2, 2, 4, 2, 4>;
using CfgDown = GemmCfg<2, 2, 4, 2, 4>;
static_assert(CfgGateUp::WM == 2 && CfgDown::WM == 2,
              "ExpertInfo::rb counts fragments per wave row for two wave rows (kTileGran = 64)");

template <typename C, bool GATE_UP>
static hipError_t launch_gemm(const uint4 *a, const uint4 *w, const float *ba, const float *bb,
                              const DispatchBuffers &d, void *out, int K, int N, int E, float limit,
                              int mt_cap, hipStream_t s) {
  const int nb_total = (GATE_UP ? 2 * N : N) / kRowBlock;
  const int n_ct = (nb_total + C::TILE_NB - 1) / C::TILE_NB;
  const int grid = ((mt_cap * n_ct + 7) / 8) * 8;
  grouped_gemm_kernel<C, GATE_UP><<<grid, C::THREADS, 0, s>>>(a, w, ba, bb, d.info, d.totals, out, K,
                                                              N, E, limit);
  return hipGetLastError();
}

hipError_t launch_gate_up(const uint16_t *xg, const uint16_t *w1, const float *b1g, const float *b1u,
                          const DispatchBuffers &d, uint16_t *act, int H, int IM, int E, float limit,
                          int mt_cap, hipStream_t s) {
  return launch_gemm<CfgGateUp, true>(reinterpret_cast<const uint4 *>(xg),
                                      reinterpret_cast<const uint4 *>(w1), b1g, b1u, d, act, H, IM,
                                      E, limit, mt_cap, s);
}

hipError_t launch_down(const uint16_t *act, const uint16_t *w2, const float *b2,
                       const DispatchBuffers &d, float *y, int H, int IM, int E, int mt_cap,
                       hipStream_t s) {
  return launch_gemm<CfgDown, false>(reinterpret_cast<const uint4 *>(act),
                                     reinterpret_cast<const uint4 *>(w2), b2, nullptr, d, y, IM, H, E,
                                     0.f, mt_cap, s);
}

}  // namespace moe
