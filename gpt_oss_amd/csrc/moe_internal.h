// Internal declarations shared by the host side of the C-ABI and the gfx950
// kernels.  Not installed; the public interface is include/moe_abi.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/moe_abi.h"

namespace moe {

constexpr int kTopK = 4;        // EXPERT_PER_TOKEN, common/defines.h:27
constexpr int kRowBlock = 32;   // rows of one MFMA fragment (v_mfma_f32_32x32x16_bf16)
constexpr int kFragK = 16;      // reduction depth of one fragment
constexpr int kFragBytes = 1024;  // 64 lanes x 8 bf16
constexpr int kTileRows = 256;  // tallest row tile of the grouped GEMMs
constexpr int kTileGran = 32;   // an expert's segment of padded rows is a multiple of one row block
constexpr float kAlpha = 1.702f;  // run.cpp:709

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

struct LayerWeights {
  uint16_t *wr = nullptr;  // router weight, bf16 in the operand order of the f64 MFMA
  float *br = nullptr;     // router bias, padded experts = -inf
  uint16_t *w1 = nullptr;  // gate_up weight, bf16 MFMA fragments, gate/up blocks paired
  float *b1g = nullptr;    // gate bias [E, IM]
  float *b1u = nullptr;    // up bias   [E, IM]
  uint16_t *w2 = nullptr;  // down weight, bf16 MFMA fragments
  float *b2 = nullptr;     // down bias [E, H]
  bool uploaded = false;
};

// ---- kernel launchers (defined in the .hip files) ----

hipError_t launch_pack_router(const float *w_src, const float *b_src, uint16_t *wr, float *br,
                              int E, int E_pad, int H, hipStream_t s);
hipError_t launch_pack_weight(const float *src, uint16_t *dst, int rows, int cols, bool gate_up,
                              hipStream_t s);
hipError_t launch_pack_bias(const float *src, float *dst_a, float *dst_b, int n, bool deinterleave,
                            hipStream_t s);

hipError_t launch_router(const uint16_t *x, const int *pos, const uint16_t *wr, const float *br,
                         int T, int H, int E, int E_pad, float *score, int *topk_i, float *topk_v,
                         hipStream_t s);

struct DispatchBuffers {
  int *blk_counts;    // [n_blk, E]
  int *offsets;       // [E+1]   exclusive scan of valid rows
  int *perm;          // [A]     position -> assignment id
  int *rowmap;        // [A_pad] padded position -> assignment id, -1 = padding
  int *inv;           // [A]     assignment id -> padded position, -1 = inactive
  ExpertInfo *info;   // [E]
  int *totals;        // [4]: total row tiles, total padded rows, total assignments
  int a_pad_cap;      // capacity of rowmap in rows
};
hipError_t launch_dispatch(const int *topk_i, const int *pos, int T, int E, const DispatchBuffers &d,
                           hipStream_t s);
hipError_t launch_gather(const uint16_t *x, const DispatchBuffers &d, uint16_t *xg, int T, int H,
                         int rb_cap, hipStream_t s);

hipError_t launch_gate_up(const uint16_t *xg, const uint16_t *w1, const float *b1g, const float *b1u,
                          const DispatchBuffers &d, uint16_t *act, int H, int IM, int E, float limit,
                          int mt_cap, hipStream_t s);
hipError_t launch_down(const uint16_t *act, const uint16_t *w2, const float *b2,
                       const DispatchBuffers &d, float *y, int H, int IM, int E, int mt_cap,
                       hipStream_t s);
hipError_t launch_combine(const float *y, const int *inv, const float *topk_v, const int *pos,
                          float *out, int T, int H, int accumulate, hipStream_t s);

}  // namespace moe
