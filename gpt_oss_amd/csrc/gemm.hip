// Grouped expert GEMMs on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16,
// fp32 accumulate).  Replaces mlp1_kernel / mlp1_120b_kernel
// (matmul/matmul.cpp:1023-1465) with the clamped SwiGLU in the epilogue
// (utility/utility.cpp:1108-1125; formula of run.cpp:709-726) and
// mlp2_kernel_noatomic / mlp2_120b_kernel (matmul/matmul.cpp:1470-1914).
//
// Data layout.  The weights and the activation between the two GEMMs are kept
// as ready-made MFMA fragments of 1 KB (64 lanes x 8 bf16, see pack.hip and the
// gate_up epilogue), ordered [row block of 32][k block of 16]: every global load
// is a contiguous 16 bytes per lane and is already in register order.  The row
// operand of gate_up is the token rows themselves, bf16 row-major, found through
// the dispatch's row map: there is no gathered copy (gemm_tile_gl for the large
// batches, the GATHER form of gemm_tile for the small ones).
//
// Tiling.  A workgroup of NW waves owns a tile of (RBT*32) rows x
// (NW*NBW*32) columns of one expert.  The waves split the columns only: each
// wave keeps RBT x NBW accumulators of 32x32 over all rows of the tile, RBT =
// 1..8 following the expert's row count (see build_plan in dispatch.hip), so a ragged
// segment pads to at most 31 rows and MFMA work follows the real rows.
//
// Feeding the matrix cores.  A step of 32 k needs 32 KB per CU, and one CU
// takes data in from L2 at about 45 GB/s with 100 KB in flight and 55-60 GB/s
// with 200 KB, so the design keeps many bytes in flight:
//   * the row operand (shared by all waves) goes straight into an R-stage LDS
//     ring by DMA (global_load_lds_dwordx4), R-1 steps ahead of the MFMAs;
//   * the column operand is private to a wave in this layout, so it never
//     touches LDS: it is loaded into an R-slot ring of VGPRs, R-1 steps ahead.
// The full-height configuration runs R = 4 (3 steps x 32 KB = 96 KB in flight
// per CU: measured against 3, 5, 6 and 7, a deeper ring gains nothing in the
// main loop and costs the time its longer fill takes at the start of every
// tile, 0.7 % of the layer per stage at 4096 tokens; with 3 the main loop
// starves); the small-batch configuration, a stream of weights through two or
// three workgroups per CU, runs R = 7.  These loads
// complete in the order they were issued, so waiting for "all but the newest n"
// (s_waitcnt vmcnt(n)) picks out exactly the step that is needed next and
// leaves the later ones in flight (the GATHER variant of gemm_tile counts
// differently, see there).
//
// Tile order.  Workgroup ids are dealt round-robin to the 8 XCDs, each with
// its own L2.  Logical tile ids are laid out (expert, group of up to four row
// tiles, column tile, row tile) with the row tile fastest, and XCD x takes a
// contiguous range of them (see build_plan and write_expert_tiles: about an
// eighth by estimated cost): the tiles an XCD runs at one time share a few row
// tiles of the expert and a few column slabs of its weights.  (Batches of at most 64 tokens
// have no tile table at all: see DIRECT at the kernel.)
#include <type_traits>
#include <utility>

#include "moe_internal.h"

namespace moe {

template <int V>
using IC = std::integral_constant<int, V>;

// f(IC<0>{}), f(IC<1>{}), ..., f(IC<N-1>{})
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
  (f(IC<I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// run.cpp:709-726: gate clamped from above, up clamped on both sides, then
// gate * sigmoid(alpha * gate) * (up + 1).  u1 is up + 1 already (the 1 rides
// in the accumulator's start value together with the bias).
__device__ __forceinline__ float swiglu_shifted(float g, float u1, float limit) {
  constexpr float kNegAlphaLog2e = -kAlpha * 1.4426950408889634f;
  g = fminf(g, limit);
  u1 = __builtin_amdgcn_fmed3f(u1, 1.0f - limit, 1.0f + limit);
  const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(kNegAlphaLog2e * g));
  return g * s * u1;
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// two floats -> packed bf16, round to nearest even (v_cvt_pk_bf16_f32); a in the low half
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Row split of a column tile with nb_valid of its NW * NBW column blocks inside
// the matrix: 4 when a quarter of the waves have columns, 2 when half have.
__host__ __device__ inline int row_split_of(int nb_valid, int nw, int nbw) {
  const int waves = (nb_valid + nbw - 1) / nbw;
  return (nw == 4 && waves == 1) ? 4 : ((nw == 4 && waves == 2) ? 2 : 1);
}

// Maps the workgroup id to a tile (see "Tile order" above): two dependent
// loads, the XCD's range and the tile's descriptor.  Returns false for the
// surplus workgroups of the upper-bound grid.
__device__ __forceinline__ bool locate_tile(const TileDesc *__restrict__ tiles,
                                            const int *__restrict__ bounds, TileDesc &d) {
  const int bid = blockIdx.x;
  const int xcd = bid & (kXcds - 1);
  const int L = bounds[xcd] + (bid >> 3);
  if (L >= bounds[xcd + 1]) return false;
  d = tiles[L];
  return true;
}

// ---- vector-memory instructions of the main loop ----

// 16 bytes per lane from global memory straight into LDS at base + 16*lane
// (global_load_lds_dwordx4; the LDS base must be wave-uniform).
__device__ __forceinline__ void dma_to_lds_16(const uint4 *g, uint4 *lds_wave_base) {
  __builtin_amdgcn_global_load_lds(g, lds_wave_base, 16, 0, 0);
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding).
// Loads return in order, so "at most n outstanding" means "all but the newest n
// have landed".  The compiler places its own waits before the first use of
// loaded data in the same wave; these explicit ones stand before the barriers,
// where other waves are about to read what this wave's DMA wrote.
#define WAIT_VMCNT(n) \
  __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | (0x7 << 4) | (0xf << 8))

// Workgroup barrier that orders LDS traffic only.  A __syncthreads (or a
// workgroup fence) would also drain the vector-memory counter and with it the
// loads of the steps still in flight.  The memory clobber keeps the compiler
// from moving memory accesses across the barrier.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Epilogue of the gate_up GEMM: SwiGLU of the (gate, up) accumulator pairs, bf16,
// stored in the fragment order the down GEMM reads as its row operand.
template <int RBT, int RS, typename C>
__device__ __forceinline__ void gate_up_epilogue(const f32x16 (&acc)[RBT][C::NBW], void *__restrict__ outp,
                                                 int out_ld, float limit, int rb0, int rbt, int nb0,
                                                 int nb_valid, int cw, int rg, int lane) {
  constexpr int NBW = C::NBW;
  // Column blocks come in (gate, up) pairs (see pack_weight_kernel): blocks 2P
  // and 2P+1 of the product hold gate_j and up_j of j = 32P .. 32P+31 in the
  // same lane and register.  The activation goes out as bf16 in the fragment
  // order the down GEMM reads as its row operand: column j is k block j/16,
  // lane ((j%16)/8)*32 + token, element j % 8.  Registers 4g .. 4g+3 of lane
  // (token t, half h) are j = 8g + 4h .. +3: elements 4h .. 4h+3 of the
  // fragment lane (g % 2)*32 + t of k block g / 2.  One exchange between the
  // lane halves (v_permlane32_swap) per dword completes the 16 bytes of every
  // fragment lane; nothing goes through LDS.
  uint4 *act = reinterpret_cast<uint4 *>(outp);
  const int kb2_total = out_ld / kFragK;
  const int P0 = (nb0 + cw * NBW) >> 1;                // first pair of this wave
  const int pairs_valid = (nb_valid - cw * NBW) >> 1;  // >= 1 here
#pragma unroll
  for (int i = 0; i < RBT; i++) {
    const int blk = i * RS + rg;
    if (RS > 1 && blk >= rbt) break;
#pragma unroll
    for (int p = 0; p < NBW / 2; p++) {
      uint32_t pk[4][2];
#pragma unroll
      for (int g = 0; g < 4; g++)
#pragma unroll
        for (int d = 0; d < 2; d++)
          pk[g][d] = pack_bf16(
              swiglu_shifted(acc[i][2 * p][4 * g + 2 * d], acc[i][2 * p + 1][4 * g + 2 * d], limit),
              swiglu_shifted(acc[i][2 * p][4 * g + 2 * d + 1], acc[i][2 * p + 1][4 * g + 2 * d + 1],
                             limit));
      uint4 *dst = act + ((size_t)(rb0 + blk) * kb2_total + 2 * (P0 + p)) * 64 + lane;
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
        // upper lane half of registers 8kb .. 8kb+3 <-> lower lane half of 8kb+4 .. 8kb+7
        const u32x2 s0 = __builtin_amdgcn_permlane32_swap(pk[2 * kb][0], pk[2 * kb + 1][0], false, false);
        const u32x2 s1 = __builtin_amdgcn_permlane32_swap(pk[2 * kb][1], pk[2 * kb + 1][1], false, false);
        if (p < pairs_valid) dst[kb * 64] = make_uint4(s0[0], s1[0], s0[1], s1[1]);
      }
    }
  }
}

template <int R>
struct StageRing {
  uint4 *p[R];
};

// NW waves side by side over the columns, NBW column blocks per wave, R ring
// slots (LDS stages for the row operand, register slots for the column operand).
// RBM = row blocks per tile at most: it sizes the LDS stages, and with them how
// many workgroups share a CU; WAVES = waves per SIMD the registers are held to.
template <int NW_, int NBW_, int R_, int RBM_ = kTileRows / kRowBlock, int WAVES_ = 1>
struct GemmCfg {
  static constexpr int NW = NW_, NBW = NBW_, R = R_, KPS = 2;
  static constexpr int THREADS = NW * 64;
  static constexpr int WAVES = WAVES_;
  static constexpr int TILE_NB = NW * NBW;              // column blocks per tile
  static constexpr int RBT_MAX = RBM_;                   // row blocks per tile, at most
  static constexpr int STAGE = RBT_MAX * KPS * 64;       // uint4 per LDS stage (16 KB)
  static constexpr int EPI_LD = NBW * 32 + 8;            // floats per buffered output row
  static constexpr int EPI_WAVE = 32 * EPI_LD / 4;       // uint4 per wave of epilogue buffer
};

// FP4: the column operand is MXFP4 as packed by pack_fp4_kernel: per pair of
// column blocks and step of 32 k one 16-byte chunk per lane (blocks 2P and 2P+1,
// each [k block 0: 8 nibbles][k block 1: 8 nibbles] of the lane's row) and two
// scale bytes per row.  A step of 32 k is exactly one MXFP4 block, so one scale
// serves both of its k blocks.  The nibbles become bf16 MFMA operands in
// registers (v_cvt_scalef32_pk_bf16_fp4: two values and their scale per
// instruction, exact); everything else is the bf16 kernel, which then takes in
// 4.25 KB instead of 16 KB of weights per CU and step.
//
// RS (row split) > 1 serves the last column tile of a matrix whose width is not
// a multiple of the tile's: only NW / RS waves would have columns there, so the
// waves form RS groups that share those columns and split the row blocks
// (group rg takes row blocks rg, rg + RS, ...).  RBT is then the row blocks per
// wave, RBT * RS are staged per step (blocks past the tile's rbt repeat its
// last one and are not stored).
//
// GATHER (gate_up of the small-batch configuration): the row operand's DMA reads
// the token rows themselves, every lane at the address of its own row (rowmap)
// -- 32 bytes per row and instruction instead of 1 KB in one piece.  While the
// GEMM is a stream of weights that is free; on tiles 4 to 8 row blocks high the
// address work of 32 cache lines per instruction costs the main loop a quarter,
// which is why the large batches fetch whole lines (gemm_tile_gl).  Here the
// waits count DMA only (see WAIT_DMA_*).
template <int RBT, int RS, typename C, bool GATE_UP, bool FP4, bool GATHER>
__device__ __forceinline__ void gemm_tile(const uint4 *__restrict__ a_frag,  // [rb][KB][64]; GATHER: token rows [T][KB*2]
                                          const uint4 *__restrict__ b_frag,  // expert: [nb][KB][64], FP4: [nb/2][KB/2][64]
                                          const uint16_t *__restrict__ b_scale,  // FP4: expert's [nb/2][KB/2][32] byte pairs
                                          int KB, int rb0, int rbt, int nb0, int nb_valid,
                                          // the part of the reduction this workgroup sums: steps (of 32 k)
                                          // [ks_begin, ks_begin + ks_count); the bias goes in with the first
                                          int ks_begin, int ks_count,
                                          const int *__restrict__ rowmap,    // GATHER: padded row -> assignment
                                          int map_rb0,                       // row block that rowmap[0] belongs to
                                          const float *__restrict__ bias_a,  // gate / down bias (expert)
                                          const float *__restrict__ bias_b,  // up bias (expert)
                                          void *__restrict__ outp, int out_ld, float limit,
                                          // One __restrict__ pointer per LDS stage: after
                                          // inlining the compiler can tell a read of one stage
                                          // from the DMA that fills another and waits only for
                                          // the fill of the stage it reads.
                                          uint4 *__restrict__ s0, uint4 *__restrict__ s1,
                                          uint4 *__restrict__ s2, uint4 *__restrict__ s3,
                                          uint4 *__restrict__ s4, uint4 *__restrict__ s5,
                                          uint4 *__restrict__ s6,
                                          // The epilogue buffers are not carved out of the
                                          // ring: the compiler would make every read of them
                                          // wait for all outstanding vector memory operations,
                                          // the epilogue's own stores included.
                                          uint4 *__restrict__ epi) {
  StageRing<C::R> ring;
  {
    uint4 *const all[7] = {s0, s1, s2, s3, s4, s5, s6};
#pragma unroll
    for (int i = 0; i < C::R; i++) ring.p[i] = all[i];
  }
  constexpr int NBW = C::NBW, KPS = C::KPS, R = C::R, NW = C::NW;
  static_assert(KPS == 2, "the step is software-pipelined as two k blocks");
  constexpr int A_CH = RBT * RS * KPS;       // 1 KB chunks of the row operand per step
  constexpr int LA = (A_CH + NW - 1) / NW;   // DMA loads per wave per step (a short last pass repeats a chunk)
  constexpr int LB = FP4 ? 2 : NBW * KPS;    // register loads per wave per step
  constexpr int LPS = LA + LB;
  static_assert(LPS * (R - 2) + LA <= 63, "vmcnt is a 6-bit counter");
  static_assert(!FP4 || NBW == 2, "an MXFP4 chunk holds the pair of column blocks of one wave");
  constexpr int NM = RBT * NBW;              // MFMAs per k block
  constexpr int DEC = FP4 ? NBW : 0;         // decode items per k block (one column block each)
  constexpr int SIDE1 = (RBT + LB + DEC + NM - 1) / NM;  // side items per MFMA, k block 0
  constexpr int SIDE2 = (LA + RBT + DEC + NM - 1) / NM;  // ... k block 1
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  static_assert(NW % RS == 0 && RBT * RS <= C::RBT_MAX, "row split");
  const int cw = RS == 1 ? w : w % (NW / RS);  // the wave's place among the columns
  const int rg = RS == 1 ? 0 : w / (NW / RS);  // ... and among the row groups

  // The accumulators start from the bias (the up half of gate_up from bias + 1,
  // see swiglu_shifted).  gate_up computes the transposed product (weights as
  // the MFMA's first operand): register q of lane l is then weight row
  // 8*(q/4) + 4*(l/32) + q%4 of its block and token l % 32.  down computes the
  // product as it is: register q is token 8*(q/4) + 4*(l/32) + q%4, lane l
  // column l % 32.  The bias loads go out first and are consumed after the
  // pipeline's loads have been issued.
  static_assert(!GATE_UP || NBW % 2 == 0, "gate and up blocks of a pair must sit in one wave");
  float4 bias_g[NBW / 2 + 1][4], bias_u[NBW / 2 + 1][4];
  float bias_d[NBW];
  if (GATE_UP) {
    // a wave past the matrix's last column (last column tile only) reads the
    // last valid pair's bias: the expert's bias vector ends there
    const int P_last = ((nb0 + nb_valid) >> 1) - 1;
    const int P0 = (nb0 + cw * NBW) >> 1;
#pragma unroll
    for (int p = 0; p < NBW / 2; p++) {
      const int P = min(P0 + p, P_last);
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int j = kRowBlock * P + 8 * g + 4 * (lane >> 5);
        bias_g[p][g] = *reinterpret_cast<const float4 *>(bias_a + j);
        bias_u[p][g] = *reinterpret_cast<const float4 *>(bias_b + j);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < NBW; j++)
      bias_d[j] = ks_begin == 0 ? bias_a[kRowBlock * (nb0 + min(cw * NBW + j, nb_valid - 1)) + (lane & 31)] : 0.f;
  }
  f32x16 acc[RBT][NBW];

  const int steps_total = KB / KPS;
  const int n_steps = ks_count;
  const uint4 *a_src = a_frag + ((size_t)rb0 * KB + ks_begin * KPS) * 64 + lane;
  // GATHER: per DMA of a step, this lane's place in its token's row (16-byte
  // units: a row is KB * 2 of them, a k block 2, the lane's half of it 1).
  // Padding rows read token 0; their products are never used.
  uint32_t lane_off[LA];
  if (GATHER) {
#pragma unroll
    for (int m = 0; m < LA; m++) {
      const int c = min(m * NW + w, A_CH - 1);
      const int blk = RS == 1 ? c / KPS : min(c / KPS, rbt - 1);
      const int a = rowmap[(rb0 - map_rb0 + blk) * kRowBlock + (lane & 31)];
      const int tok = a >= 0 ? a / kTopK : 0;
      lane_off[m] = (uint32_t)tok * (uint32_t)(KB * 2) + (ks_begin * KPS + c % KPS) * 2 + (lane >> 5);
    }
  }
  // Column blocks past the end of the matrix (last column tile only) re-load
  // the last valid block; their products are never stored.
  const uint4 *b_src[NBW];
  const uint16_t *s_src = nullptr;
  if (FP4) {
    const size_t pair = (size_t)((nb0 + min(cw * NBW, nb_valid - NBW)) >> 1);
    b_src[0] = b_frag + (pair * steps_total + ks_begin) * 64 + lane;
    s_src = b_scale + (pair * steps_total + ks_begin) * 32 + (lane & 31);
  } else {
#pragma unroll
    for (int j = 0; j < NBW; j++)
      b_src[j] = b_frag + ((size_t)(nb0 + min(cw * NBW + j, nb_valid - 1)) * KB + ks_begin * KPS) * 64 + lane;
  }

  // Row operand: chunk c of a step (c = pass*NW + wave) is row block c / KPS, k block c % KPS.
  auto issue_a = [&](uint4 *st, int ks, int m) {
    const int c = min(m * NW + w, A_CH - 1);
    const int blk = RS == 1 ? c / KPS : min(c / KPS, rbt - 1);
    if (GATHER) {
      dma_to_lds_16(a_frag + lane_off[m] + ks * (KPS * 2), st + c * 64);
    } else {
      dma_to_lds_16(a_src + ((size_t)blk * KB + ks * KPS + c % KPS) * 64, st + c * 64);
    }
  };
  // Column operand: register m of a slot is column block m / KPS, k block m % KPS.
  // FP4: load 0 of a slot is the chunk of nibbles, load 1 the two scale bytes.
  u32x4 bq[R][FP4 ? 1 : LB];
  uint32_t bsc[R];
  auto issue_b = [&](int slot, int ks, int m) {
    if (FP4) {
      if (m == 0) {
        bq[slot][0] = *reinterpret_cast<const u32x4 *>(b_src[0] + (size_t)ks * 64);
      } else {
        bsc[slot] = s_src[(size_t)ks * 32];
      }
    } else {
      bq[slot][m] = *reinterpret_cast<const u32x4 *>(b_src[m / KPS] + (size_t)(ks * KPS + m % KPS) * 64);
    }
  };
  // FP4: the decoded operands of the step at hand, [column block][k block].
  // Those of k block 0 are decoded during the previous step's second half,
  // those of k block 1 during this step's first half.
  bf16x8 bdec[NBW][KPS];
  auto decode = [&](int slot, int j, int kk) {
    const float scale = __uint_as_float(((bsc[slot] >> (8 * j)) & 0xffu) << 23);  // 2^(s - 127)
    const uint32_t nib = bq[slot][0][j * KPS + kk];
    const bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 0);
    const bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 1);
    const bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 2);
    const bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 3);
    bdec[j][kk] = bf16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  };
  // Two register sets of row fragments: while the MFMAs of one k block run, the
  // fragments of the next are read from LDS.
  bf16x8 fa[2][RBT];
  auto read_a = [&](const uint4 *st, int kk, int buf, int i) {
    fa[buf][i] = __builtin_bit_cast(bf16x8, st[((i * RS + rg) * KPS + kk) * 64 + lane]);
  };
  auto mma = [](bf16x8 rows, bf16x8 colv, f32x16 c) {
    return GATE_UP ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(colv, rows, c, 0, 0, 0)
                   : __builtin_amdgcn_mfma_f32_32x32x16_bf16(rows, colv, c, 0, 0, 0);
  };
  // column operand of (slot, column block j, k block kk)
  auto cols_of = [&](int slot, int j, int kk) {
    if constexpr (FP4) {
      return bdec[j][kk];
    } else {
      return __builtin_bit_cast(bf16x8, bq[slot][j * KPS + kk]);
    }
  };
  static_assert(R >= 3 && R <= 7, "up to seven stage arrays are passed in");
  // "Step s of the row operand has landed" as a bound on the vector-memory
  // counter.  The loads are issued in the order A(0) B(0) A(1) B(1) ... and
  // complete in that order, so all but the newest n outstanding means step s has
  // landed with n = everything issued behind it.  With the scattered DMA of the
  // GATHER form and the mixed count, wrong token rows were once seen in this
  // configuration (several workgroups per CU, ring of 7), different from run to
  // run; the cause was never established (the same scattered DMA with the mixed
  // count gives the same bits in every run on the large batches).  Here the
  // bound counts the DMAs behind step s only, which holds whatever the register
  // loads do and costs nothing while the tile is a stream of weights.
  constexpr int WAIT_DMA_FILL = GATHER ? LA * (R - 1) : LPS * (R - 2) + LA;  // A(0), A(0..R-1) issued
  constexpr int WAIT_DMA_STEP = GATHER ? LA * (R - 2) : LPS * (R - 2);       // A(ks+1) at step ks

  // Issue order per wave: A(0) B(0) A(1) B(1) ... ; at the top of step ks the row
  // operand is issued through step ks+R-1 and the column operand through ks+R-2
  // (step indices past the tile's last are clamped to it).
  const int last = n_steps - 1;
#pragma unroll
  for (int s = 0; s < R - 1; s++) {
#pragma unroll
    for (int m = 0; m < LA; m++) issue_a(ring.p[s], min(s, last), m);
#pragma unroll
    for (int m = 0; m < LB; m++) issue_b(s, min(s, last), m);
    __builtin_amdgcn_sched_barrier(0);  // the counted waits rely on this issue order
  }
  if (GATE_UP) {
#pragma unroll
    for (int p = 0; p < NBW / 2; p++)
#pragma unroll
      for (int g = 0; g < 4; g++)
#pragma unroll
        for (int i = 0; i < RBT; i++) {
          const float4 bg = bias_g[p][g], bu = bias_u[p][g];
          acc[i][2 * p][4 * g + 0] = bg.x; acc[i][2 * p][4 * g + 1] = bg.y;
          acc[i][2 * p][4 * g + 2] = bg.z; acc[i][2 * p][4 * g + 3] = bg.w;
          acc[i][2 * p + 1][4 * g + 0] = bu.x + 1.0f; acc[i][2 * p + 1][4 * g + 1] = bu.y + 1.0f;
          acc[i][2 * p + 1][4 * g + 2] = bu.z + 1.0f; acc[i][2 * p + 1][4 * g + 3] = bu.w + 1.0f;
        }
  } else {
#pragma unroll
    for (int j = 0; j < NBW; j++)
#pragma unroll
      for (int i = 0; i < RBT; i++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[i][j][q] = bias_d[j];
  }
#pragma unroll
  for (int m = 0; m < LA; m++) issue_a(ring.p[R - 1], min(R - 1, last), m);
  WAIT_VMCNT(WAIT_DMA_FILL);
  lds_barrier();
#pragma unroll
  for (int i = 0; i < RBT; i++) read_a(ring.p[0], 0, 0, i);
  if (FP4) {
#pragma unroll
    for (int j = 0; j < NBW; j++) decode(0, j, 0);
  }

  // Step ks, slot u = ks % R:
  //   [MFMAs of k block 0 | read row fragments of k block 1, load B(ks+R-1) into slot u-1]
  //   wait until step ks+1 has arrived, barrier
  //   [MFMAs of k block 1 | DMA A(ks+R) into stage u, read row fragments of step ks+1]
  // The side work is spread over the MFMAs so that it issues in their shadow.
  // Every step is the same straight code with the same count in its wait: the
  // refills of the tile's last R-1 steps, for which there is nothing left to
  // load, load its last step again (cache hits that nobody reads) instead of
  // being skipped.  Skipping them costs more: with refills guarded at run time
  // the waits can no longer be counted and the last six steps took twice their
  // time (-3.4 % on gate_up, -4.9 % on down with the loads kept).  The wave
  // ends with those loads in flight; s_endpgm waits for them.
  auto step = [&](auto u_c, int ks) {
    constexpr int u = decltype(u_c)::value;
    const uint4 *cur = ring.p[u];
    const int ks_b = min(ks + R - 1, last);
    const int ks_a = min(ks + R, last);
#pragma unroll
    for (int m = 0; m < NM; m++) {
#pragma unroll
      for (int t = m * SIDE1; t < (m + 1) * SIDE1; t++) {
        if (t < RBT) {
          read_a(cur, 1, 1, t);
        } else if (t < RBT + LB) {
          issue_b((u + R - 1) % R, ks_b, t - RBT);
        } else if (t < RBT + LB + DEC) {
          decode(u, t - RBT - LB, 1);
        }
      }
      acc[m / NBW][m % NBW] = mma(fa[0][m / NBW], cols_of(u, m % NBW, 0), acc[m / NBW][m % NBW]);
      __builtin_amdgcn_sched_barrier(0);
    }
    WAIT_VMCNT(WAIT_DMA_STEP);
    lds_barrier();  // step ks+1 is complete in LDS; every wave is done with stage u
    const uint4 *nxt = ring.p[(u + 1) % R];
#pragma unroll
    for (int m = 0; m < NM; m++) {
#pragma unroll
      for (int t = m * SIDE2; t < (m + 1) * SIDE2; t++) {
        if (t < LA) {
          issue_a(ring.p[u], ks_a, t);
        } else if (t < LA + RBT) {
          read_a(nxt, 0, 0, t - LA);
        } else if (t < LA + RBT + DEC) {
          decode((u + 1) % R, t - LA - RBT, 0);  // landed: the wait above covers it
        }
      }
      acc[m / NBW][m % NBW] = mma(fa[1][m / NBW], cols_of(u, m % NBW, 1), acc[m / NBW][m % NBW]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int ks0 = 0;
  for (; ks0 + R <= n_steps; ks0 += R)
    static_for<R>([&](auto u_c) { step(u_c, ks0 + decltype(u_c)::value); });
  static_for<R - 1>([&](auto u_c) {
    if (ks0 + decltype(u_c)::value < n_steps) step(u_c, ks0 + decltype(u_c)::value);
  });

  // Epilogue.
  if (cw * NBW >= nb_valid) return;  // a wave without columns (last column tile only)
  if (GATE_UP) {
    gate_up_epilogue<RBT, RS, C>(acc, outp, out_ld, limit, rb0, rbt, nb0, nb_valid, cw, rg, lane);
  } else if constexpr (C::RBT_MAX == 2) {
    // Small-batch configuration: the rows go out straight from the accumulators
    // (register q of lane l is token 8*(q/4) + 4*(l/32) + q%4, column l % 32: a
    // store writes two rows of 128 contiguous bytes).  No LDS buffer, so that a
    // third workgroup fits a CU; at full tile height the two forms take the same
    // time.
    static_assert(RS == 1, "the small-batch configuration has no row split");
    float *y = reinterpret_cast<float *>(outp);
    const int n = lane & 31;
    const int rsub = 4 * (lane >> 5);
#pragma unroll
    for (int i = 0; i < RBT; i++) {
      const size_t row0 = (size_t)(rb0 + i) * kRowBlock;
#pragma unroll
      for (int j = 0; j < NBW; j++) {
        if (cw * NBW + j >= nb_valid) continue;
        float *dst = y + row0 * out_ld + kRowBlock * (nb0 + cw * NBW + j) + n;
#pragma unroll
        for (int q = 0; q < 16; q++) dst[(size_t)(8 * (q >> 2) + rsub + (q & 3)) * out_ld] = acc[i][j][q];
      }
    }
  } else {
    constexpr int LD = C::EPI_LD;  // +8 floats keep the two lane halves on different banks
    float *y = reinterpret_cast<float *>(outp);
    float *ef = reinterpret_cast<float *>(epi + w * C::EPI_WAVE);
    const int n = lane & 31;
    const int rsub = 4 * (lane >> 5);
    const int col0 = kRowBlock * (nb0 + cw * NBW);
#pragma unroll
    for (int i = 0; i < RBT; i++) {
      const int blk = i * RS + rg;
      if (RS > 1 && blk >= rbt) break;
#pragma unroll
      for (int j = 0; j < NBW; j++)
#pragma unroll
        for (int q = 0; q < 16; q++) {
          const int r = 8 * (q >> 2) + rsub + (q & 3);
          ef[r * LD + 32 * j + n] = acc[i][j][q];
        }
      const size_t row0 = (size_t)(rb0 + blk) * kRowBlock;
#pragma unroll
      for (int t = 0; t < NBW * 4; t++) {
        const int idx = t * 64 + lane;
        const int r = idx / (NBW * 8);
        const int c4 = idx % (NBW * 8);
        const float4 v = *reinterpret_cast<const float4 *>(ef + r * LD + 4 * c4);
        if (cw * NBW + c4 / 8 < nb_valid)
          *reinterpret_cast<float4 *>(y + (row0 + r) * out_ld + col0 + 4 * c4) = v;
      }
    }
  }
}

// double stages of the row operand in gemm_tile_gl (3: 96 KB of LDS, 4: 128 KB)
constexpr int kLineStages = 4;

// gate_up of the large batches without a gathered copy of the routed rows: the
// row operand's DMA reads the token rows themselves, WHOLE CACHE LINES at a time.
// One instruction fetches 8 rows x 128 bytes (64 k); a scattered DMA that takes
// 32 bytes of 32 rows per instruction (the small-batch form in gemm_tile) costs
// the main loop a quarter more, and 64 bytes of 16 rows an eighth.
//
// So the row operand is staged in double steps: a double stage holds 64 k of
// all rows of the tile (two 16 KB arrays: row blocks 0-3 and 4-7), R2 of them
// form the ring, and the refill comes every other step.  Wave w fetches rows
// 8w .. 8w+7 of every row block; inside its kilobyte a lane holds one 16-byte
// piece of one of the 8 rows, and WHICH is chosen so that (a) the four lanes of
// a quad read 64 contiguous bytes of one row and (b) the MFMA operand reads
// (lane = row, all lanes the same piece) find 8 consecutive rows on the 8
// different 16-byte slots of 128 bytes of LDS and 16 consecutive rows on the 16
// of 256 bytes: quad Q = 4 * (row / 2) + 2 * (half of the line ^ w % 2) + row % 2,
// and lane j of the quad holds piece (j - row / 2) mod 4 of that half.
//
// The column operand keeps its ring of RB register slots of one step each.
// Loads are issued in the order  B(0) B(1) B(2) A2(0) A2(1) A2(2) A2(3) | step 0:
// B(3) | step 1: B(4) A2(4) | step 2: B(5) | step 3: B(6) A2(5) | ...  (R2 = RB =
// 4).  The counted wait in the middle of a step leaves the newest 2 LB + LA2
// loads in flight (see gemm_tile for the assumption): that covers A2(d+1), which
// an odd step 2d+1 needs, and B(ks+1), which every step's successor needs.  Even
// steps need no barrier: they read a double stage that landed before the
// previous odd step's barrier and refill nothing.
template <int RBT, int RS, typename C, bool FP4>
__device__ __forceinline__ void gemm_tile_gl(const uint4 *__restrict__ x_rows,  // token rows [T][KB * 2] of 16 bytes
                                             const uint4 *__restrict__ b_frag,
                                             const uint16_t *__restrict__ b_scale, int KB, int rb0, int rbt,
                                             int nb0, int nb_valid, const int *__restrict__ rowmap,
                                             const float *__restrict__ bias_a,
                                             const float *__restrict__ bias_b, void *__restrict__ outp,
                                             int out_ld, float limit, uint4 *__restrict__ s0,
                                             uint4 *__restrict__ s1, uint4 *__restrict__ s2,
                                             uint4 *__restrict__ s3, uint4 *__restrict__ s4,
                                             uint4 *__restrict__ s5, uint4 *__restrict__ s6,
                                             uint4 *__restrict__ s7) {
  constexpr int NBW = C::NBW, KPS = C::KPS, RB = C::R, NW = C::NW, R2 = kLineStages;
  static_assert(KPS == 2 && NW == 4 && RB == 4 && C::RBT_MAX == 8 && (RS == 1 || RS == 2), "shape of the line gather");
  constexpr int NB = RBT * RS;                // row blocks staged per step
  constexpr int LA2 = NB;                     // DMA loads per wave and double step: one per row block
  constexpr int LB = FP4 ? 2 : NBW * KPS;     // register loads per wave and step
  static_assert(!FP4 || NBW == 2, "an MXFP4 chunk holds the pair of column blocks of one wave");
  constexpr int NM = RBT * NBW;               // MFMAs per k block
  constexpr int DEC = FP4 ? NBW : 0;
  static_assert(R2 >= 3, "with 2 double stages an odd step would have to wait for all but 2 * LB loads");
  constexpr int WAIT_FILL = (R2 - 1) * LA2;  // the loads behind A2(0) in the first filling
  constexpr int WAIT_MID = 2 * LB + LA2;                                     // see the steps
  static_assert(WAIT_FILL <= 63 && WAIT_MID <= 63, "vmcnt is a 6-bit counter");
  uint4 *const arr[8] = {s0, s1, s2, s3, s4, s5, s6, s7};
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cw = RS == 1 ? w : w % (NW / RS);
  const int rg = RS == 1 ? 0 : w / (NW / RS);

  float4 bias_g[NBW / 2][4], bias_u[NBW / 2][4];
  {
    const int P_last = ((nb0 + nb_valid) >> 1) - 1;
    const int P0 = (nb0 + cw * NBW) >> 1;
#pragma unroll
    for (int p = 0; p < NBW / 2; p++) {
      const int P = min(P0 + p, P_last);
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int j = kRowBlock * P + 8 * g + 4 * (lane >> 5);
        bias_g[p][g] = *reinterpret_cast<const float4 *>(bias_a + j);
        bias_u[p][g] = *reinterpret_cast<const float4 *>(bias_b + j);
      }
    }
  }
  f32x16 acc[RBT][NBW];
  const int n_steps = KB / KPS;  // even: the depth is a multiple of 64
  const int last = n_steps - 1, last_d = n_steps / 2 - 1;

  // this lane's source in a double step of row block m: its token's row and its piece of the line.
  // The row map is asked for here; the answer is used after the column operand's
  // first loads have gone out (below), so that its latency costs the tile nothing.
  uint32_t lane_src[LA2];
  int lane_piece;
  {
    const int Q = lane >> 2, j = lane & 3;  // quad Q of the kilobyte: row 2 * (Q / 4) + Q % 2, one half of its line
    const int row8 = 2 * (Q >> 2) + (Q & 1);
    lane_piece = 4 * (((Q >> 1) & 1) ^ (w & 1)) + ((j - (Q >> 2)) & 3);
#pragma unroll
    for (int m = 0; m < LA2; m++) {
      const int blk = RS == 1 ? m : min(m, rbt - 1);
      lane_src[m] = (uint32_t)rowmap[(rb0 + blk) * kRowBlock + 8 * w + row8];
    }
  }
  // where this lane finds its operand of (parity of the step, k block) inside a row block's 4 KB
  int lane_rd[2][KPS];
  {
    const int r = lane & 31, h = lane >> 5, sub = r >> 3, row8 = r & 7;
#pragma unroll
    for (int par = 0; par < 2; par++)
#pragma unroll
      for (int kk = 0; kk < KPS; kk++)
        lane_rd[par][kk] = sub * 64 + (4 * (row8 >> 1) + 2 * (par ^ (sub & 1)) + (row8 & 1)) * 4 +
                           ((kk * 2 + h + (row8 >> 1)) & 3);
  }
  const uint4 *b_src[NBW];
  const uint16_t *s_src = nullptr;
  if (FP4) {
    const size_t pair = (size_t)((nb0 + min(cw * NBW, nb_valid - NBW)) >> 1);
    b_src[0] = b_frag + pair * n_steps * 64 + lane;
    s_src = b_scale + pair * n_steps * 32 + (lane & 31);
  } else {
#pragma unroll
    for (int j = 0; j < NBW; j++)
      b_src[j] = b_frag + (size_t)(nb0 + min(cw * NBW + j, nb_valid - 1)) * KB * 64 + lane;
  }

  // double step jd of row block m into double stage slot d
  auto issue_a2 = [&](int d, int jd, int m) {
    dma_to_lds_16(x_rows + lane_src[m] + jd * 8, arr[2 * d + (m >= 4 ? 1 : 0)] + ((m & 3) * 4 + w) * 64);
  };
  u32x4 bq[RB][FP4 ? 1 : LB];
  uint32_t bsc[RB];
  auto issue_b = [&](int slot, int ks, int m) {
    if (FP4) {
      if (m == 0) {
        bq[slot][0] = *reinterpret_cast<const u32x4 *>(b_src[0] + (size_t)ks * 64);
      } else {
        bsc[slot] = s_src[(size_t)ks * 32];
      }
    } else {
      bq[slot][m] = *reinterpret_cast<const u32x4 *>(b_src[m / KPS] + (size_t)(ks * KPS + m % KPS) * 64);
    }
  };
  bf16x8 bdec[NBW][KPS];
  auto decode = [&](int slot, int j, int kk) {
    const float scale = __uint_as_float(((bsc[slot] >> (8 * j)) & 0xffu) << 23);
    const uint32_t nib = bq[slot][0][j * KPS + kk];
    const bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 0);
    const bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 1);
    const bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 2);
    const bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, scale, 3);
    bdec[j][kk] = bf16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  };
  bf16x8 fa[2][RBT];
  // fragment of the wave's row block i from double stage slot d
  auto read_a = [&](int d, int par, int kk, int buf, int i) {
    const uint4 *st = arr[2 * d + (i * RS >= 4 ? 1 : 0)];
    fa[buf][i] = __builtin_bit_cast(bf16x8, st[(((i * RS + rg) & 3) * 4) * 64 + lane_rd[par][kk]]);
  };
  auto mma = [](bf16x8 rows, bf16x8 colv, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(colv, rows, c, 0, 0, 0);
  };
  auto cols_of = [&](int slot, int j, int kk) {
    if constexpr (FP4) {
      return bdec[j][kk];
    } else {
      return __builtin_bit_cast(bf16x8, bq[slot][j * KPS + kk]);
    }
  };

  // one double step of the row operand / one step of the column operand, all of the wave's loads
  auto issue_a2_all = [&](int d, int jd) {
#pragma unroll
    for (int m = 0; m < LA2; m++) issue_a2(d, min(jd, last_d), m);
  };
  auto issue_b_all = [&](int slot, int ks) {
#pragma unroll
    for (int m = 0; m < LB; m++) issue_b(slot, min(ks, last), m);
  };
  // first filling: B(0) .. B(RB-2), then (the row map has answered meanwhile) A2(0) .. A2(R2-1)
#pragma unroll
  for (int k = 0; k < RB - 1; k++) issue_b_all(k, k);
  __builtin_amdgcn_sched_barrier(0);  // the counted waits rely on this issue order
#pragma unroll
  for (int m = 0; m < LA2; m++) {
    const int a = (int)lane_src[m];
    const int tok = a >= 0 ? a / kTopK : 0;  // padding rows read token 0; their products are never used
    lane_src[m] = (uint32_t)tok * (uint32_t)(KB * 2) + lane_piece;
  }
#pragma unroll
  for (int k = 0; k < R2 - 1; k++) issue_a2_all(k, k);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int p = 0; p < NBW / 2; p++)
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
      for (int i = 0; i < RBT; i++) {
        const float4 bg = bias_g[p][g], bu = bias_u[p][g];
        acc[i][2 * p][4 * g + 0] = bg.x; acc[i][2 * p][4 * g + 1] = bg.y;
        acc[i][2 * p][4 * g + 2] = bg.z; acc[i][2 * p][4 * g + 3] = bg.w;
        acc[i][2 * p + 1][4 * g + 0] = bu.x + 1.0f; acc[i][2 * p + 1][4 * g + 1] = bu.y + 1.0f;
        acc[i][2 * p + 1][4 * g + 2] = bu.z + 1.0f; acc[i][2 * p + 1][4 * g + 3] = bu.w + 1.0f;
      }
  issue_a2_all(R2 - 1, R2 - 1);
  WAIT_VMCNT(WAIT_FILL);
  lds_barrier();
#pragma unroll
  for (int i = 0; i < RBT; i++) read_a(0, 0, 0, 0, i);
  if (FP4) {
#pragma unroll
    for (int j = 0; j < NBW; j++) decode(0, j, 0);
  }

  // Step ks = 2 jd + par, u = ks mod PERIOD: column slot u % RB, double stage (u / 2) % R2.
  auto step = [&](auto u_c, int ks) {
    constexpr int u = decltype(u_c)::value;
    constexpr int slot = u % RB, d = (u / 2) % R2, par = u % 2;
    constexpr int LAX = par ? LA2 : 0;             // the refill comes with the odd steps
    constexpr int dn = par ? (d + 1) % R2 : d;     // the next step's double stage
    constexpr int SIDE1 = (RBT + LB + DEC + NM - 1) / NM;
    constexpr int SIDE2 = (LAX + RBT + DEC + NM - 1) / NM;
    const int ks_b = min(ks + RB - 1, last);
    const int jd_a = min(ks / 2 + R2, last_d);
#pragma unroll
    for (int m = 0; m < NM; m++) {
#pragma unroll
      for (int t = m * SIDE1; t < (m + 1) * SIDE1; t++) {
        if (t < RBT) {
          read_a(d, par, 1, 1, t);
        } else if (t < RBT + LB) {
          issue_b((slot + RB - 1) % RB, ks_b, t - RBT);
        } else if (t < RBT + LB + DEC) {
          decode(slot, t - RBT - LB, 1);
        }
      }
      acc[m / NBW][m % NBW] = mma(fa[0][m / NBW], cols_of(slot, m % NBW, 0), acc[m / NBW][m % NBW]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // Every step says in its middle what has landed, as a count: all but the
    // column loads of the last two steps and the double step issued between
    // them.  An odd step needs A2(jd+1), which lies further back, for the
    // fragment reads that follow; every step needs B(ks+1) for its successor's
    // first MFMA, and with the count given here the compiler adds no wait of its
    // own (left to itself it waits for ALL loads before some of the steps).
    WAIT_VMCNT(WAIT_MID);
    if constexpr (par == 1) {
      lds_barrier();  // double step jd+1 is complete in LDS; every wave is done with double stage d
    } else {
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int m = 0; m < NM; m++) {
#pragma unroll
      for (int t = m * SIDE2; t < (m + 1) * SIDE2; t++) {
        if (t < LAX) {
          issue_a2(d, jd_a, t);
        } else if (t < LAX + RBT) {
          read_a(dn, par ^ 1, 0, 0, t - LAX);
        } else if (t < LAX + RBT + DEC) {
          decode((slot + 1) % RB, t - LAX - RBT, 0);
        }
      }
      acc[m / NBW][m % NBW] = mma(fa[1][m / NBW], cols_of(slot, m % NBW, 1), acc[m / NBW][m % NBW]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  constexpr int PERIOD = R2 == 3 ? 12 : 2 * R2;  // a multiple of 2 * R2 and of RB
  static_assert(PERIOD % RB == 0 && PERIOD % (2 * R2) == 0, "one unrolled round serves both rings");
  int ks0 = 0;
  for (; ks0 + PERIOD <= n_steps; ks0 += PERIOD)
    static_for<PERIOD>([&](auto u_c) { step(u_c, ks0 + decltype(u_c)::value); });
  static_for<PERIOD - 1>([&](auto u_c) {
    if (ks0 + decltype(u_c)::value < n_steps) step(u_c, ks0 + decltype(u_c)::value);
  });

  if (cw * NBW >= nb_valid) return;  // a wave without columns (last column tile only)
  gate_up_epilogue<RBT, RS, C>(acc, outp, out_ld, limit, rb0, rbt, nb0, nb_valid, cw, rg, lane);
}

// DIRECT (small-batch configuration only): there is no plan.  A workgroup is
// one column tile of one expert (see the mapping below); its 256 threads look at one
// assignment of the batch each and find the expert's rows with a ballot (see
// DirectIds).  An expert without rows ends its workgroups here.
template <typename C, bool GATE_UP, bool FP4, bool GATHER, bool DIRECT = false>
__global__ __launch_bounds__(C::THREADS, C::WAVES) void grouped_gemm_kernel(
    const uint4 *__restrict__ a_frag, const uint4 *__restrict__ w_frag,
    const uint16_t *__restrict__ w_scale,
    const float *__restrict__ bias_a, const float *__restrict__ bias_b,
    const TileDesc *__restrict__ tiles, const int *__restrict__ totals,
    const int *__restrict__ rowmap, void *__restrict__ outp, int K, int N, float limit,
    DirectIds ids, size_t split_stride) {
  static_assert(!GATHER || GATE_UP, "only the first GEMM reads token rows");
  static_assert(!DIRECT || (C::RBT_MAX * kRowBlock == kDirectSlotRows && C::THREADS == kDirectTokens * kTopK),
                "a direct batch: one thread per assignment, an expert's slot is one tile high");
  constexpr int R = C::R;
  static_assert(R <= 7, "seven stage arrays are declared below");
  __shared__ uint4 st0[C::STAGE], st1[C::STAGE], st2[C::STAGE], st3[C::STAGE], st4[C::STAGE],
      st5[C::STAGE], st6[C::STAGE], st7[C::STAGE];  // those a variant does not use take no room
  __shared__ uint4 epi[C::RBT_MAX == 2 ? 1 : C::NW * C::EPI_WAVE];  // the small-batch configuration stores directly
  const int KB = K / kFragK;
  const int nb_total = (GATE_UP ? 2 * N : N) / kRowBlock;  // weight row blocks per expert
  const int n_ct = (nb_total + C::TILE_NB - 1) / C::TILE_NB;
  TileDesc tc;
  __shared__ int direct_rows[kDirectSlotRows];  // slot row -> assignment, -1 = padding
  __shared__ int direct_cnt[C::NW];
  const int *map = rowmap;
  if constexpr (DIRECT) {
    const int tid = threadIdx.x;
    // Workgroup ids are dealt round-robin to the 8 XCDs: XCD x takes the experts
    // x, x + 8, ..., all column tiles of an expert, so that the expert's rows
    // (which every one of its column tiles reads) are fetched into one L2
    // instead of eight.
    const int xcd = blockIdx.x & (kXcds - 1), idx = blockIdx.x >> 3;
    const int e = (idx / n_ct) * kXcds + xcd;
    if (e >= ids.E) return;  // surplus workgroups of the grid (experts not a multiple of 8)
    const bool mine = direct_expert_of(ids, tid) == e;
    const unsigned long long bal = __ballot(mine);
    if ((tid & 63) == 0) direct_cnt[tid >> 6] = __popcll(bal);
    if (tid < kDirectSlotRows) direct_rows[tid] = -1;
    __syncthreads();
    int before = 0, count = 0;
#pragma unroll
    for (int ww = 0; ww < C::NW; ww++) {
      const int c = direct_cnt[ww];
      if (ww < (tid >> 6)) before += c;
      count += c;
    }
    if (count == 0) return;
    if (GATHER) {
      const int r = before + __popcll(bal & ((1ull << (tid & 63)) - 1ull));
      if (mine && r < kDirectSlotRows) direct_rows[r] = tid;
      __syncthreads();
      map = direct_rows;
    }
    tc.e = e;
    tc.nt = idx % n_ct;
    tc.rb0 = e * (kDirectSlotRows / kRowBlock);
    tc.rbt = (min(count, kDirectSlotRows) + kRowBlock - 1) / kRowBlock;
  } else {
    if (!locate_tile(tiles, totals + (GATE_UP ? kTotBoundsGateUp : kTotBoundsDown), tc)) return;
  }
  const int map_rb0 = DIRECT ? tc.rb0 : 0;
  // The down GEMM of the small-batch configuration splits the reduction over
  // gridDim.y workgroups; part p writes its sums to its own copy of the output,
  // split_stride bytes behind the one before (the combine adds the parts up).
  const int steps_total = K / (kFragK * C::KPS);
  const int ks_per = (steps_total + (int)gridDim.y - 1) / (int)gridDim.y;
  const int ks_begin = GATE_UP ? 0 : (int)blockIdx.y * ks_per;
  const int ks_count = GATE_UP ? steps_total : min(ks_per, steps_total - ks_begin);
  if (!GATE_UP) outp = static_cast<char *>(outp) + (size_t)blockIdx.y * split_stride;
  const int nb0 = tc.nt * C::TILE_NB;
  const int nb_valid = min(C::TILE_NB, nb_total - nb0);
  // per expert: bf16 nb_total * KB fragments of 1 KB; MXFP4 (nb_total/2) * (KB/2) chunks of 1 KB
  const uint4 *b_frag = w_frag + (size_t)tc.e * nb_total * KB * (FP4 ? 16 : 64);
  const uint16_t *b_scale = FP4 ? w_scale + (size_t)tc.e * nb_total * KB * 8 : nullptr;
  const float *ba = bias_a + (size_t)tc.e * N;
  const float *bb = GATE_UP ? bias_b + (size_t)tc.e * N : nullptr;
  // large batches of gate_up read the token rows by whole cache lines (gemm_tile_gl)
  constexpr bool LINES = GATHER && C::RBT_MAX == 8;
#define MOE_TILE_RS(n, rs)                                                                                    \
  do {                                                                                                        \
    if constexpr (LINES && rs <= 2) {                                                                         \
      gemm_tile_gl<n, rs, C, FP4>(a_frag, b_frag, b_scale, KB, tc.rb0, tc.rbt, nb0, nb_valid, rowmap, ba, bb, \
                                  outp, N, limit, st0, st1, st2, st3, st4, st5, st6, st7);                    \
    } else {                                                                                                  \
      gemm_tile<n, rs, C, GATE_UP, FP4, GATHER>(a_frag, b_frag, b_scale, KB, tc.rb0, tc.rbt, nb0, nb_valid,   \
                                                ks_begin, ks_count, map, map_rb0, ba, bb, outp, N, limit,     \
                                                st0, st1, st2, st3, st4, st5, st6, epi);                      \
    }                                                                                                         \
  } while (0)
#define MOE_TILE(n) MOE_TILE_RS(n, 1)
  if constexpr (C::RBT_MAX == 8) {
    // the last column tile, when only a quarter or half of the waves have columns in it
    const int rs = row_split_of(nb_valid, C::NW, C::NBW);
    if (!GATE_UP && rs == 4) {  // gate_up comes in (gate, up) pairs of pairs: never a quarter
      if (tc.rbt <= 4) MOE_TILE_RS(1, 4); else MOE_TILE_RS(2, 4);
      return;
    }
    if (rs == 2) {
      switch ((tc.rbt + 1) >> 1) {
        case 1: MOE_TILE_RS(1, 2); break;
        case 2: MOE_TILE_RS(2, 2); break;
        case 3: MOE_TILE_RS(3, 2); break;
        default: MOE_TILE_RS(4, 2); break;
      }
      return;
    }
    switch (tc.rbt) {
      case 1: MOE_TILE(1); break;
      case 2: MOE_TILE(2); break;
      case 3: MOE_TILE(3); break;
      case 4: MOE_TILE(4); break;
      case 5: MOE_TILE(5); break;
      case 6: MOE_TILE(6); break;
      case 7: MOE_TILE(7); break;
      default: MOE_TILE(8); break;
    }
  } else {
    static_assert(C::RBT_MAX == 2, "tile heights of the small-batch configuration");
    if (tc.rbt == 1) MOE_TILE(1); else MOE_TILE(2);
  }
#undef MOE_TILE
#undef MOE_TILE_RS
}

// 4 waves, one per SIMD, each 256 rows x 64 columns (8 x 2 accumulators = all
// 256 accumulation registers); 256 x 256 tiles; 4 ring slots.
using CfgGemm = GemmCfg<4, 2, 4>;
static_assert(CfgGemm::RBT_MAX * kRowBlock == kTileRows && CfgGemm::TILE_NB == kGemmTileNb,
              "tile plan of build_plan");
// Batches of at most 64 tokens: no expert has more than 64 rows, every tile is
// one or two row blocks high and the GEMMs are a stream of weights.  What
// limits that stream is the bytes one CU keeps in flight, so the same kernel is
// built with LDS stages for two row blocks and registers for two waves per
// SIMD, and several workgroups share a CU.
using CfgGemmSmall = GemmCfg<4, 2, 7, 2, 2>;
using CfgGemmSmallFp4 = GemmCfg<4, 2, 7, 2, 3>;
constexpr int kSmallBatchTokens = CfgGemmSmall::RBT_MAX * kRowBlock;

// w_scale == nullptr: w holds bf16 fragments; otherwise w holds MXFP4 chunks and
// w_scale their scale bytes (pack_fp4_kernel).
// CF: the configuration of the MXFP4 instance (its column operand's ring takes a
// third of the registers, so the small-batch down GEMM, which has no LDS buffer
// for its output, can be held to three waves per SIMD; holding gate_up to the
// same bound changes nothing in its register count and cost it 3 us per call).
template <typename C, bool GATE_UP, bool GATHER = false, bool DIRECT = false, typename CF = C>
static hipError_t launch_gemm(const uint4 *a, const uint4 *w, const uint16_t *w_scale, const float *ba,
                              const float *bb, const DispatchBuffers &d, void *out, int K, int N,
                              float limit, int mt_cap, const DirectIds &direct, int k_split,
                              size_t split_stride, hipStream_t s) {
  const int nb_total = (GATE_UP ? 2 * N : N) / kRowBlock;
  const int n_ct = (nb_total + C::TILE_NB - 1) / C::TILE_NB;
  const dim3 grid(DIRECT ? kXcds * ((direct.E + kXcds - 1) / kXcds) * n_ct : kXcds * xcd_tile_cap(mt_cap * n_ct),
                  GATE_UP ? 1 : k_split);
  const TileDesc *tiles = GATE_UP ? d.tiles_gate_up : d.tiles_down;
  if (w_scale) {
    grouped_gemm_kernel<CF, GATE_UP, true, GATHER, DIRECT><<<grid, CF::THREADS, 0, s>>>(
        a, w, w_scale, ba, bb, tiles, d.totals, d.rowmap, out, K, N, limit, direct, split_stride);
  } else {
    grouped_gemm_kernel<C, GATE_UP, false, GATHER, DIRECT><<<grid, C::THREADS, 0, s>>>(
        a, w, nullptr, ba, bb, tiles, d.totals, d.rowmap, out, K, N, limit, direct, split_stride);
  }
  return hipGetLastError();
}

hipError_t launch_gate_up(const uint16_t *x, const void *w1, const uint16_t *w1_scale, const float *b1g,
                          const float *b1u, const DispatchBuffers &d, uint16_t *act, int H, int IM,
                          float limit, int mt_cap, int max_rows, const DirectIds &direct, hipStream_t s) {
  static_assert(kSmallBatchTokens == kSmallBatchRows, "small_batch() and the small-batch configuration");
  const uint4 *w = reinterpret_cast<const uint4 *>(w1);
  const uint4 *rows = reinterpret_cast<const uint4 *>(x);
  if (direct.topk_i)
    return launch_gemm<CfgGemmSmall, true, true, true>(rows, w, w1_scale, b1g, b1u, d, act, H, IM, limit,
                                                       mt_cap, direct, 1, 0, s);
  // either way the row operand is read from the token rows: 32 bytes of 32 rows per
  // instruction in the small-batch configuration, whole lines of 8 rows otherwise
  if (small_batch(max_rows))
    return launch_gemm<CfgGemmSmall, true, true>(rows, w, w1_scale, b1g, b1u, d, act, H, IM, limit, mt_cap,
                                                 direct, 1, 0, s);
  return launch_gemm<CfgGemm, true, true>(rows, w, w1_scale, b1g, b1u, d, act, H, IM, limit, mt_cap, direct, 1, 0,
                                          s);
}

hipError_t launch_down(const uint16_t *act, const void *w2, const uint16_t *w2_scale, const float *b2,
                       const DispatchBuffers &d, float *y, int H, int IM, int mt_cap, int max_rows,
                       const DirectIds &direct, int k_split, size_t split_stride, hipStream_t s) {
  const uint4 *a = reinterpret_cast<const uint4 *>(act);
  const uint4 *w = reinterpret_cast<const uint4 *>(w2);
  // The smallest batches: a workgroup is one stream of weights, and the few
  // experts such a batch reaches leave most CUs without one.  Two workgroups
  // per tile then sum half of the reduction each into their own copy of the
  // rows (down_k_split; the combine adds the two parts).
  const int ks = small_batch(max_rows) ? k_split : 1;
  if (direct.topk_i)
    return launch_gemm<CfgGemmSmall, false, false, true, CfgGemmSmallFp4>(a, w, w2_scale, b2, nullptr, d, y, IM, H,
                                                                          0.f, mt_cap, direct, ks, split_stride, s);
  if (small_batch(max_rows))
    return launch_gemm<CfgGemmSmall, false, false, false, CfgGemmSmallFp4>(a, w, w2_scale, b2, nullptr, d, y, IM, H,
                                                                           0.f, mt_cap, direct, ks, split_stride, s);
  return launch_gemm<CfgGemm, false>(a, w, w2_scale, b2, nullptr, d, y, IM, H, 0.f, mt_cap, direct, 1, 0, s);
}

}  // namespace moe
