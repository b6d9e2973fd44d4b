// Weight ingest: fp32 host layout of the reference (run.cpp:234-247) -> bf16
// (round to nearest even, as utility.cpp:509/:534/:610 do at upload) in the
// fragment order the gfx950 MFMA kernels read.  Replaces
// pack_fp32_to_bf16_matmul (utility/utility.cpp:558-622) and the per-expert
// host loops of getp_run.cpp:259-293 / expert.cpp:971-1009.
#include "moe_internal.h"

namespace moe {

__device__ __forceinline__ float bf16_round(float f) {
  return __uint_as_float((uint32_t)f32_to_bf16_rne(f) << 16);
}

// One fragment = 32 output rows x 16 reduction elements, stored as 64 lanes x
// 8 bf16: lane l holds row (l % 32), k = 8*(l / 32) .. +7 -- the B-operand
// register layout of v_mfma_f32_32x32x16_bf16.  Fragments are ordered
// [row block][k block].  With gate_up set, row block 2p holds the gate rows
// (source rows 2j) and row block 2p+1 the up rows (source rows 2j+1) of
// j = 32p .. 32p+31, so that a lane's gate and up accumulators line up and the
// SwiGLU epilogue needs no exchange between lanes.
//
// The packed matrix has rows_p x cols_p elements (multiples of 64, see
// padded_dim); what lies outside the source's rows x cols is zero, so that a
// padded reduction adds nothing and a padded output column is its bias alone.
__global__ void pack_weight_kernel(const float *__restrict__ src, uint4 *__restrict__ dst, int rows,
                                   int cols, int rows_p, int cols_p, int gate_up) {
  const int kb_total = cols_p / kFragK;
  const size_t n_chunks = (size_t)(rows_p / kRowBlock) * kb_total * 64;
  for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < n_chunks;
       c += (size_t)gridDim.x * blockDim.x) {
    const int lane = (int)(c & 63);
    const size_t frag = c >> 6;
    const int kb = (int)(frag % kb_total);
    const int nb = (int)(frag / kb_total);
    const int n = lane & 31;
    const int k0 = kb * kFragK + 8 * (lane >> 5);
    const int row = gate_up ? 2 * (kRowBlock * (nb >> 1) + n) + (nb & 1) : kRowBlock * nb + n;
    uint4 o = make_uint4(0u, 0u, 0u, 0u);
    if (row >= rows || k0 >= cols) {  // cols is a multiple of 8: a piece lies inside or outside
      dst[c] = o;
      continue;
    }
    const float4 *p = reinterpret_cast<const float4 *>(src + (size_t)row * cols + k0);
    const float4 a = p[0], b = p[1];
    o.x = f32_to_bf16_rne(a.x) | ((uint32_t)f32_to_bf16_rne(a.y) << 16);
    o.y = f32_to_bf16_rne(a.z) | ((uint32_t)f32_to_bf16_rne(a.w) << 16);
    o.z = f32_to_bf16_rne(b.x) | ((uint32_t)f32_to_bf16_rne(b.y) << 16);
    o.w = f32_to_bf16_rne(b.z) | ((uint32_t)f32_to_bf16_rne(b.w) << 16);
    dst[c] = o;
  }
}

// MXFP4 ingest (export_model_bin/gpt-oss-20b/export_model_bin.py:86-123): a
// row of `cols` weights is cols/32 blocks of 16 bytes plus one scale byte per
// block; byte b of a block holds element 2b in its low nibble and element 2b+1
// in its high nibble; a nibble indexes {0, .5, 1, 1.5, 2, 3, 4, 6} and their
// negatives, and the scale byte s multiplies by 2^(s - 127).  The weights stay
// in this format on the device, re-ordered for the GEMMs that decode them in
// registers (gemm_tile with FP4).  Per pair of row blocks (2P, 2P+1) and step of 32 k (one
// MXFP4 block): a 16-byte chunk per lane l = (row n = l % 32, half h = l / 32),
//   bytes 0-3   row of block 2P,   k block 0: elements 8h .. 8h+7  = source bytes 4h .. 4h+3
//   bytes 4-7   row of block 2P,   k block 1: elements 16+8h ..    = source bytes 8+4h ..
//   bytes 8-15  the same for block 2P+1,
// and for every n the two scale bytes (block 2P, block 2P+1).  With gate_up set
// the row blocks are the (gate, up) pairs of pack_weight_kernel.
// Rows and steps of the padded matrix (rows_p x cols_p) outside the source are
// zero nibbles with scale byte 127 (2^0).
__global__ void pack_fp4_kernel(const uint8_t *__restrict__ blocks, const uint8_t *__restrict__ scales,
                                uint4 *__restrict__ wq, uint16_t *__restrict__ ws, int rows, int cols,
                                int rows_p, int cols_p, int gate_up) {
  const int steps = cols_p / 32, src_steps = cols / 32;
  const int pairs = rows_p / (2 * kRowBlock);
  const size_t n_chunks = (size_t)pairs * steps * 64;
  for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < n_chunks;
       c += (size_t)gridDim.x * blockDim.x) {
    const int lane = (int)(c & 63);
    const size_t ps = c >> 6;
    const int step = (int)(ps % steps);
    const int P = (int)(ps / steps);
    const int n = lane & 31, h = lane >> 5;
    uint32_t o[4];
    uint32_t sc = 0;
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int nb = 2 * P + j;
      const int row = gate_up ? 2 * (kRowBlock * (nb >> 1) + n) + (nb & 1) : kRowBlock * nb + n;
      if (row >= rows || step >= src_steps) {
        o[2 * j + 0] = o[2 * j + 1] = 0u;
        sc |= 127u << (8 * j);
        continue;
      }
      const size_t g = (size_t)row * src_steps + step;
      const uint8_t *src = blocks + g * 16;
      o[2 * j + 0] = *reinterpret_cast<const uint32_t *>(src + 4 * h);
      o[2 * j + 1] = *reinterpret_cast<const uint32_t *>(src + 8 + 4 * h);
      sc |= (uint32_t)scales[g] << (8 * j);
    }
    wq[c] = make_uint4(o[0], o[1], o[2], o[3]);
    if (h == 0) ws[((size_t)P * steps + step) * 32 + n] = (uint16_t)sc;
  }
}

// Router weight as bf16 in the operand order of v_mfma_f32_16x16x32_bf16:
// [expert block of 16][k chunk of 32][lane][s], s = 0..7: lane l holds expert
// 16*nb + (l % 16) and k = 32*kc + 8*(l / 16) + s, the same split of a chunk's
// k over the lanes as the activations are loaded with.  Experts beyond E are
// zero weight with bias -inf; the selection skips them by index.
__global__ void pack_router_kernel(const float *__restrict__ w, const float *__restrict__ b,
                                   uint16_t *__restrict__ wr, float *__restrict__ br, int E,
                                   int E_pad, int H) {
  const int kc_total = H / 32;
  const size_t n = (size_t)(E_pad / 16) * kc_total * 64 * 8;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const int s = (int)(i & 7);
    const int lane = (int)((i >> 3) & 63);
    const size_t f = i >> 9;
    const int kc = (int)(f % kc_total);
    const int nb = (int)(f / kc_total);
    const int e = nb * 16 + (lane & 15);
    const int k = kc * 32 + 8 * (lane >> 4) + s;
    wr[i] = e < E ? f32_to_bf16_rne(w[(size_t)e * H + k]) : (uint16_t)0;
  }
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t < E_pad) br[t] = t < E ? bf16_round(b[t]) : -INFINITY;
}

// Biases are kept as fp32 holding bf16-rounded values (the reference keeps
// them as bf16, expert.cpp:906-930).  deinterleave: src[2j] -> a[j], src[2j+1] -> b[j].
// The source holds rows of `len` values, the destination rows of len_p >= len
// (of len_p / 2 for each half when de-interleaving); the padding is zero.
__global__ void pack_bias_kernel(const float *__restrict__ src, float *__restrict__ a,
                                 float *__restrict__ b, int n_rows, int len, int len_p, int deinterleave) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_rows * len_p) return;
  const int r = i / len_p, j = i % len_p;
  const float v = j < len ? bf16_round(src[(size_t)r * len + j]) : 0.f;
  if (deinterleave) {
    const size_t o = (size_t)r * (len_p / 2) + (j >> 1);
    if (j & 1) b[o] = v; else a[o] = v;
  } else {
    a[i] = v;
  }
}

hipError_t launch_pack_router(const float *w_src, const float *b_src, uint16_t *wr, float *br, int E,
                              int E_pad, int H, hipStream_t s) {
  pack_router_kernel<<<512, 256, 0, s>>>(w_src, b_src, wr, br, E, E_pad, H);
  return hipGetLastError();
}

hipError_t launch_pack_weight(const float *src, uint16_t *dst, int rows, int cols, int rows_p, int cols_p,
                              bool gate_up, hipStream_t s) {
  pack_weight_kernel<<<2048, 256, 0, s>>>(src, reinterpret_cast<uint4 *>(dst), rows, cols, rows_p, cols_p,
                                          gate_up ? 1 : 0);
  return hipGetLastError();
}

hipError_t launch_pack_fp4(const uint8_t *blocks, const uint8_t *scales, uint8_t *wq, uint16_t *ws,
                           int rows, int cols, int rows_p, int cols_p, bool gate_up, hipStream_t s) {
  pack_fp4_kernel<<<2048, 256, 0, s>>>(blocks, scales, reinterpret_cast<uint4 *>(wq), ws, rows, cols,
                                       rows_p, cols_p, gate_up ? 1 : 0);
  return hipGetLastError();
}

hipError_t launch_pack_bias(const float *src, float *dst_a, float *dst_b, int n_rows, int len, int len_p,
                            bool deinterleave, hipStream_t s) {
  const int n = n_rows * len_p;
  pack_bias_kernel<<<(n + 255) / 256, 256, 0, s>>>(src, dst_a, dst_b, n_rows, len, len_p,
                                                   deinterleave ? 1 : 0);
  return hipGetLastError();
}

}  // namespace moe
