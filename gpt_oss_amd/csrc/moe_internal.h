// Internal declarations shared by the host side of the C-ABI and the gfx950
// kernels.  Not installed; the public interface is include/moe_abi.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/moe_abi.h"

namespace moe {

// Records the text of a failure for moe_last_error() on the calling thread and
// returns `code` (defined with the C-ABI's host side).
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// float -> bf16 bits, round to nearest even; a NaN stays a NaN
// (/opt/rocm/include/hip/amd_detail/amd_hip_bfloat16.h:96-131).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if (~u & 0x7f800000u) {
    u += 0x7fffu + ((u >> 16) & 1u);
  } else if (u & 0xffffu) {
    u |= 0x10000u;
  }
  return (uint16_t)(u >> 16);
}

constexpr int kTopK = 4;        // EXPERT_PER_TOKEN, common/defines.h:27
constexpr int kRowBlock = 32;   // rows of one MFMA fragment (v_mfma_f32_32x32x16_bf16)
constexpr int kFragK = 16;      // reduction depth of one fragment
constexpr int kFragBytes = 1024;  // 64 lanes x 8 bf16
constexpr int kTileRows = 256;  // tallest row tile of the grouped GEMMs
constexpr int kTileGran = 32;   // an expert's segment of padded rows is a multiple of one row block
constexpr float kAlpha = 1.702f;  // run.cpp:709

// Work split of the grouped GEMMs over the 8 XCDs (each has an L2 of its own).
// Tiles are numbered (expert, group of row tiles, column tile, row tile of the
// group), row tile fastest; XCD x takes the tiles [bounds[x], bounds[x+1]), a
// range of about an eighth of the estimated cost.  (Cutting the last tiles of a range into smaller pieces, so
// that its CUs run dry together, was measured and does not pay: the pieces are
// less efficient than what they save.)
constexpr int kGemmTileNb = 8;  // column blocks (of 32) per tile of the grouped GEMMs
constexpr int kRowTileGroup = 4;  // row tiles of one expert that run side by side (see write_expert_tiles)
constexpr int kXcds = 8;
// estimated cost of a tile: kCostPerTile + kCostPerRowBlock * row blocks.  The
// fixed part (4 row blocks' worth) was fitted on measured runs with even,
// Zipf-skewed and 128-expert routing; it stands for the column operand, which
// a tile streams in full however few rows it has.
constexpr int kCostPerTile = 32;
constexpr int kCostPerRowBlock = 8;
// layout of DispatchBuffers::totals
constexpr int kTotTiles = 0, kTotRows = 1, kTotAssign = 2;
constexpr int kTotBoundsGateUp = 4;            // 9 ints
constexpr int kTotBoundsDown = 4 + kXcds + 1;  // 9 ints
constexpr int kTotInts = 4 + 2 * (kXcds + 1);

// Most tiles one XCD can be given out of `total`: the balancing never moves a
// boundary further than this, so that the launch grid can be sized on the host.
__host__ __device__ inline int xcd_tile_cap(int total) { return (total + 7) / 8 + (total + 15) / 16 + 1; }

// Per-expert record written by the scan kernel and read by the GEMMs.
struct ExpertInfo {
  int row0;       // first padded row of the expert's segment (multiple of 32)
  int rows;       // valid rows (assignments) of the expert
  int n_mt;       // number of row tiles
  int rb;         // row blocks of the expert's shorter tiles (0..8)
  int tile_base;  // number of row tiles of all lower experts
  int extra;      // its first `extra` tiles have rb + 1 row blocks
  int pad_[2];
};

// One tile of a grouped GEMM, looked up by its number in the tile sequence.
// Written by the scan kernel for both GEMMs, so that a GEMM workgroup finds its
// work with one load instead of a binary search over the experts (a chain of
// dependent global loads in front of every tile).
struct TileDesc {
  int e;    // expert
  int rb0;  // first row block of the tile in the padded row space
  int rbt;  // its row blocks (1..8)
  int nt;   // column tile
};

struct LayerWeights {
  uint16_t *wr = nullptr;  // router weight, bf16 in the operand order of v_mfma_f32_16x16x32_bf16
  float *br = nullptr;     // router bias [E_pad] (padded experts = -inf), then the two floats of rstat
  uint16_t *w1 = nullptr;  // gate_up weight, bf16 MFMA fragments, gate/up blocks paired
  float *b1g = nullptr;    // gate bias [E, IM]
  float *b1u = nullptr;    // up bias   [E, IM]
  uint16_t *w2 = nullptr;  // down weight, bf16 MFMA fragments
  float *b2 = nullptr;     // down bias [E, H]
  // Expert matrices kept as MXFP4 instead (moe_upload_layer_mxfp4): 16-byte
  // chunks of nibbles and two scale bytes per row, pair of row blocks and 32 k
  // (see pack_fp4_kernel); w1/w2 are then not allocated.
  uint8_t *w1q = nullptr, *w2q = nullptr;
  uint16_t *w1s = nullptr, *w2s = nullptr;
  float *rms_w = nullptr;  // weight of the RMS norm in front of the layer [H] (bf16 values), optional
  bool uploaded = false;
};

// ---- kernel launchers (defined in the .hip files) ----

hipError_t launch_pack_router(const float *w_src, const float *b_src, uint16_t *wr, float *br,
                              int E, int E_pad, int H, hipStream_t s);
// The grouped GEMMs work on matrices whose sides are multiples of 64 (a double
// step of the reduction, a pair of column blocks).  Sizes that are multiples of
// 32 only are padded to that inside the library: zero weights and biases at
// upload, zero columns of the routed rows per call (launch_pad_rows).  The
// reference pads its packed weights likewise (utility/utility.cpp:558-622).
constexpr int kDimGran = 64;
inline int padded_dim(int n) { return (n + kDimGran - 1) / kDimGran * kDimGran; }
// rows x cols (source) -> rows_p x cols_p (packed, zero outside the source)
hipError_t launch_pack_weight(const float *src, uint16_t *dst, int rows, int cols, int rows_p, int cols_p,
                              bool gate_up, hipStream_t s);
hipError_t launch_pack_fp4(const uint8_t *blocks, const uint8_t *scales, uint8_t *wq, uint16_t *ws,
                           int rows, int cols, int rows_p, int cols_p, bool gate_up, hipStream_t s);
// n_rows rows of len values -> rows of len_p (each half len_p / 2 when de-interleaving)
hipError_t launch_pack_bias(const float *src, float *dst_a, float *dst_b, int n_rows, int len, int len_p,
                            bool deinterleave, hipStream_t s);
hipError_t launch_pad_rows(const uint16_t *x, uint16_t *xp, int T, int H, int Hp, hipStream_t s);

// rstat: two floats written by launch_router_stats at upload (largest 2-norm of
// an expert's router weights, largest bias magnitude), the inputs of the error
// bound that decides which tokens need exact fp64 logits.
hipError_t launch_router_stats(const float *w_src, const float *b_src, int E, int H, float *rstat,
                               hipStream_t s);
hipError_t launch_router(const uint16_t *x, const int *pos, const uint16_t *wr, const float *br,
                         const float *rstat, int T, int H, int E, int E_pad, float *score, int *topk_i,
                         float *topk_v, hipStream_t s);

struct DispatchBuffers {
  int *blk_counts;    // [n_blk, E]
  int *offsets;       // [E+1]   exclusive scan of valid rows
  int *perm;          // [A]     position -> assignment id
  int *rowmap;        // [A_pad] padded position -> assignment id, -1 = padding
  int *inv;           // [A]     assignment id -> padded position, -1 = inactive
  ExpertInfo *info;   // [E]
  int *totals;        // [kTotInts]: total row tiles, padded rows, assignments; XCD bounds of both GEMMs
  int a_pad_cap;      // capacity of rowmap in rows
  TileDesc *tiles_gate_up;  // [tile_cap_gate_up] tile sequence of the gate_up GEMM
  TileDesc *tiles_down;     // [tile_cap_down]    ... of the down GEMM
  int tile_cap_gate_up, tile_cap_down;
};
hipError_t launch_dispatch(const int *topk_i, const int *pos, int T, int E, int n_ct_gate_up,
                           int n_ct_down, const DispatchBuffers &d, hipStream_t s);

// Batches of at most kDirectTokens tokens run without a dispatch pass: the 256
// threads of a workgroup hold one assignment each, so every workgroup of the
// GEMMs and of the combine reads the batch's expert ids itself and finds its
// rows with a ballot.  Expert e owns the padded rows [e * kDirectSlotRows,
// (e + 1) * kDirectSlotRows); inside them its assignments stand in ascending
// order, as the dispatch kernels place them.  Requires that no expert is given
// more than kDirectSlotRows assignments.  topk_i == nullptr: not in use, the
// plan of launch_dispatch is.
constexpr int kDirectTokens = 64;
constexpr int kDirectSlotRows = 64;
struct DirectIds {
  const int *topk_i;  // [T, 4]
  const int *pos;     // [T] or nullptr
  int T, E;
};
// expert of assignment a by the rule of the dispatch kernels: -1 past the batch,
// for a row with pos < 0 and for an id outside [0, E)
__device__ __forceinline__ int direct_expert_of(const DirectIds &d, int a) {
  if (a >= d.T * kTopK) return -1;
  const int id = d.topk_i[a];                      // both loads go out together
  const int ps = d.pos ? d.pos[a / kTopK] : 0;
  return ps >= 0 && id >= 0 && id < d.E ? id : -1;
}
inline bool direct_plan_fits(int T, int max_rows, int E, int a_pad_cap) {
  return T <= kDirectTokens && max_rows <= kDirectSlotRows && kDirectSlotRows * E <= a_pad_cap;
}
// gate_up reads the routed token rows of x itself, through rowmap; there is no
// gathered copy.  Batches in which no expert has more than kSmallBatchRows rows
// run the small-batch configuration of both GEMMs.
constexpr int kSmallBatchRows = 64;
inline bool small_batch(int max_rows) { return max_rows <= kSmallBatchRows; }
// Parts the down GEMM's reduction is split into (each part writes its own copy
// of the output rows, which the combine adds up): two in the small-batch
// configuration while the experts a batch of T tokens can reach have at most
// one tile per CU between them -- a tile is one stream of weights there, and a
// CU takes in two to three such streams at once --, else one.  Measured with
// MXFP4 weights at 32 experts: a layer call at 1 token 54.8 -> 47.9 us, at 4
// tokens 65 -> 62; from 8 tokens on the split gains nothing (the first GEMM's
// workgroups already fill the CUs when the second starts).
constexpr int kSmallBatchKSplit = 2;
constexpr int kCus = 256;
inline int down_k_split(int max_rows, int inter_padded, int hidden_padded, int E, int T) {
  if (!small_batch(max_rows) || inter_padded < 64) return 1;
  const int n_ct = (hidden_padded / kRowBlock + kGemmTileNb - 1) / kGemmTileNb;
  const long long reach = (long long)T * kTopK < E ? (long long)T * kTopK : E;
  return reach * n_ct <= kCus ? kSmallBatchKSplit : 1;
}
// The rows a small batch can reach in the padded row space: every expert's
// rows rounded up to 32, or its fixed slot of 64 rows without a dispatch pass.
inline int small_batch_pad_rows(int E) {
  const int planned = kSmallBatchRows * kTopK + kTileGran * E, slots = kDirectSlotRows * E;
  return planned > slots ? planned : slots;
}
hipError_t launch_gate_up(const uint16_t *x, const void *w1, const uint16_t *w1_scale, const float *b1g,
                          const float *b1u, const DispatchBuffers &d, uint16_t *act, int H, int IM,
                          float limit, int mt_cap, int max_rows, const DirectIds &direct, hipStream_t s);
// k_split: parts of the reduction (down_k_split); split_stride: bytes between the copies of y they write
hipError_t launch_down(const uint16_t *act, const void *w2, const uint16_t *w2_scale, const float *b2,
                       const DispatchBuffers &d, float *y, int H, int IM, int mt_cap, int max_rows,
                       const DirectIds &direct, int k_split, size_t split_stride, hipStream_t s);
// direct.topk_i != nullptr: the rows of y are found from the ids (inv is not read)
// ldy: floats per row of y (the padded hidden size).  y_parts copies of y lie
// part_stride floats apart (the parts of a split reduction, see down_k_split);
// a row of the down projection is their sum, added in that order.
hipError_t launch_combine(const float *y, int ldy, int y_parts, size_t part_stride, const int *inv,
                          const float *topk_v, const int *pos, float *out, int T, int H, int accumulate,
                          const DirectIds &direct, hipStream_t s);
hipError_t launch_combine_residual(const float *y, int ldy, int y_parts, size_t part_stride, const int *inv,
                                   const float *topk_v, const int *pos, uint16_t *x, int T, int H,
                                   const DirectIds &direct, hipStream_t s);
hipError_t launch_rmsnorm(const uint16_t *x, const float *weight, const int *pos, uint16_t *t_out,
                          int T, int H, hipStream_t s);

}  // namespace moe
