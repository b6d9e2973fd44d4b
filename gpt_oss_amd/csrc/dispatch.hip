// Token -> expert dispatch: LDS histogram, prefix sum, stable permutation and
// the tile plan of the grouped GEMMs, and the combine that ends the layer.  Replaces
// count_expert_assignments_kernel, exclusive_scan_small_kernel and
// build_expert_assignments_kernel (utility/utility.cpp:1058-1106, :758-777),
// whose order inside an expert segment is the order global atomics happen to
// resolve in (utility.cpp:1101).  Here the order is fixed: inside a segment
// assignments are sorted by token index, then by slot.  No global atomics.
#include "moe_internal.h"

namespace moe {

constexpr int kDispThreads = 256;  // tokens per workgroup in count / scatter

// Pass 1: per-workgroup histogram of expert ids over active rows.  Also resets
// rowmap and perm to -1 (a fill kernel rather than a memset so that the call
// sequence can be captured in a graph).
__global__ __launch_bounds__(kDispThreads) void dispatch_count_kernel(
    const int *__restrict__ topk_i, const int *__restrict__ pos, int T, int E,
    int *__restrict__ blk_counts, int *__restrict__ rowmap, int a_pad_cap, int *__restrict__ perm) {
  __shared__ int hist[256];
  const int tid = threadIdx.x;
  hist[tid] = 0;
  __syncthreads();
  const int t = blockIdx.x * kDispThreads + tid;
  if (t < T && !(pos && pos[t] < 0)) {
    const int4 ids = *reinterpret_cast<const int4 *>(topk_i + (size_t)t * kTopK);
    const int id[kTopK] = {ids.x, ids.y, ids.z, ids.w};
#pragma unroll
    for (int k = 0; k < kTopK; k++) {
      if (id[k] >= 0 && id[k] < E) atomicAdd(&hist[id[k]], 1);
    }
  }
  __syncthreads();
  if (tid < E) blk_counts[(size_t)blockIdx.x * E + tid] = hist[tid];
  for (int i = blockIdx.x * kDispThreads + tid; i < a_pad_cap; i += gridDim.x * kDispThreads)
    rowmap[i] = -1;
  for (int i = blockIdx.x * kDispThreads + tid; i < T * kTopK; i += gridDim.x * kDispThreads)
    perm[i] = -1;
}

// The plan of one batch from the experts' row counts (thread e holds expert e's
// count; all 256 threads of the workgroup call this together).  Returns the
// expert's first row in the padded row space.
struct PlanOut {
  int *offsets;
  ExpertInfo *info;
  int *totals;
  TileDesc *tiles_gate_up, *tiles_down;
  int tile_cap_gate_up, tile_cap_down;
};

// The tiles of expert ee in the tile sequences of both GEMMs.  An expert's row
// tiles are taken in groups of at most kRowTileGroup (sizes as even as they go);
// tile L = (expert, group, column tile, row tile of the group), row tile fastest.
// The 32 CUs of an XCD then run a few column tiles of one group at a time: the
// group's rows are fetched once per generation of tiles instead of once per
// column tile (an expert with 28 row tiles otherwise streams all its rows
// through the 4 MB L2 for each of its 23 column tiles).  Measured at 7168 tokens
// with Zipf routing: the gate_up GEMM's reads from beyond L2 3.78 -> 2.77 GB, the
// down GEMM's 1.75 -> 1.51 GB, durations unchanged; experts with up to
// kRowTileGroup row tiles (even routing at 4096 tokens) are laid out as before.
// One wave; its lanes run over the expert's tiles of both GEMMs in one sweep.
__device__ __forceinline__ void write_expert_tiles(int ee, int nmt, int rbe, int exe, int rowblk, int first,
                                                   int lane, int n_ct_gate_up, int n_ct_down,
                                                   const PlanOut &out) {
  if (nmt == 0) return;
  const int n_up = nmt * n_ct_gate_up, n = n_up + nmt * n_ct_down;
  for (int ii = lane; ii < n; ii += 64) {
    const bool g = ii >= n_up;
    const int i = g ? ii - n_up : ii;
    const int L = first * (g ? n_ct_down : n_ct_gate_up) + i;
    const int n_ct = g ? n_ct_down : n_ct_gate_up;
    const int n_grp = (nmt + kRowTileGroup - 1) / kRowTileGroup;
    const int gs = nmt / n_grp, gx = nmt - gs * n_grp;  // the first gx groups hold gs + 1 row tiles
    const int big = gx * (gs + 1) * n_ct;               // tiles of those groups
    int grp, r, gsz;
    if (i < big) {
      grp = i / ((gs + 1) * n_ct);
      r = i - grp * (gs + 1) * n_ct;
      gsz = gs + 1;
    } else {
      grp = gx + (i - big) / (gs * n_ct);
      r = (i - big) - (grp - gx) * gs * n_ct;
      gsz = gs;
    }
    const int nt = r / gsz;
    const int mt = grp * gs + min(grp, gx) + (r - nt * gsz);
    TileDesc d;
    d.e = ee;
    d.nt = nt;
    d.rbt = rbe + (mt < exe ? 1 : 0);
    d.rb0 = rowblk + mt * rbe + min(mt, exe);
    if (L < (g ? out.tile_cap_down : out.tile_cap_gate_up)) (g ? out.tiles_down : out.tiles_gate_up)[L] = d;
  }
}

// write_global: this workgroup stores the plan (offsets, per-expert records,
// totals, XCD bounds); the others only need the values returned to them.
// with_tiles: this workgroup also writes the tile tables of all experts.
__device__ __forceinline__ int build_plan(int count, int E, int n_ct_gate_up, int n_ct_down,
                                          const PlanOut &out, bool with_tiles, int *ex_count_out,
                                          int *tot_count_out = nullptr, bool write_global = true,
                                          ExpertInfo *info_out = nullptr) {
  __shared__ int sh_wave[4][4];  // [wave][quantity]: the waves' sums
  __shared__ int sh_nmt[256], sh_rb[256], sh_extra[256], sh_rowblk[256];
  __shared__ int sh_cost[257];   // exclusive prefix of the experts' cost per column tile
  __shared__ int sh_tiles[257];  // exclusive prefix of their row tiles
  __shared__ int sh_bound[2][kXcds + 1];
  const int e = threadIdx.x;
  const int lane = e & 63;
  const int w = e >> 6;
  int *offsets = out.offsets;
  ExpertInfo *info = out.info;
  int *totals = out.totals;
  const int n_rb = (count + kRowBlock - 1) / kRowBlock;
  constexpr int kTileRb = kTileRows / kRowBlock;
  const int n_mt = (n_rb + kTileRb - 1) / kTileRb;
  const int rb = n_mt ? n_rb / n_mt : 0;
  const int extra = n_mt ? n_rb - rb * n_mt : 0;
  // cost of one column tile's worth of the expert's row tiles
  const int cost = n_mt * (kCostPerTile + kCostPerRowBlock * rb) + kCostPerRowBlock * extra;
  // Exclusive prefix sums over the experts of four quantities at once: rows,
  // padded rows, row tiles, cost.  In a wave by lane shifts, across the four
  // waves through LDS.
  const int own[4] = {count, n_rb * kRowBlock, n_mt, cost};
  int incl[4] = {own[0], own[1], own[2], own[3]};
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int up = __shfl_up(incl[i], off, 64);
      if (lane >= off) incl[i] += up;
    }
  }
  if (lane == 63) {
#pragma unroll
    for (int i = 0; i < 4; i++) sh_wave[w][i] = incl[i];
  }
  __syncthreads();
  int ex[4], tot[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int below = 0, all = 0;
#pragma unroll
    for (int ww = 0; ww < 4; ww++) {
      const int v = sh_wave[ww][i];
      below += ww < w ? v : 0;
      all += v;
    }
    ex[i] = below + incl[i] - own[i];
    tot[i] = all;
  }
  const int ex_count = ex[0], ex_pad = ex[1], ex_mt = ex[2], ex_cost = ex[3];
  const int tot_count = tot[0], tot_pad = tot[1], tot_mt = tot[2], tot_cost = tot[3];
  {
    ExpertInfo inf;
    inf.row0 = ex_pad;
    inf.rows = count;
    inf.n_mt = n_mt;
    inf.rb = rb;
    inf.tile_base = ex_mt;
    inf.extra = extra;
    inf.pad_[0] = inf.pad_[1] = 0;
    if (e < E && write_global) {
      offsets[e] = ex_count;
      info[e] = inf;
    }
    if (info_out) *info_out = inf;
  }
  if (!write_global) {  // (the same for the whole workgroup)
    *ex_count_out = ex_count;
    if (tot_count_out) *tot_count_out = tot_count;
    return ex_pad;
  }
  sh_cost[e] = ex_cost;
  sh_tiles[e] = ex_mt;
  sh_nmt[e] = n_mt;
  sh_rb[e] = rb;
  sh_extra[e] = extra;
  sh_rowblk[e] = ex_pad / kRowBlock;
  if (e == 0) {
    sh_cost[256] = tot_cost;
    sh_tiles[256] = tot_mt;
    offsets[E] = tot_count;
    totals[kTotTiles] = tot_mt;
    totals[kTotRows] = tot_pad;
    totals[kTotAssign] = tot_count;
    totals[3] = 0;
  }
  __syncthreads();
  // Thread (g, x): boundary x of GEMM g = first tile at which the cost so far
  // reaches x/8 of the total (an expert's tiles taken as equally dear: their heights differ by one block at most).
  if (e < 2 * (kXcds + 1)) {
    const int g = e / (kXcds + 1), x = e % (kXcds + 1);
    const int n_ct = g ? n_ct_down : n_ct_gate_up;
    const int total_tiles = tot_mt * n_ct;
    int bound;
    if (x == 0) {
      bound = 0;
    } else if (x == kXcds) {
      bound = total_tiles;
    } else {
      const long long target = (long long)tot_cost * n_ct * x / kXcds;
      // last expert whose first tile starts at or before the target
      int lo = 0, hi = 255;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if ((long long)sh_cost[mid] * n_ct <= target) lo = mid; else hi = mid - 1;
      }
      const int c_e = sh_cost[lo + 1] - sh_cost[lo];  // > 0: the search stops on an expert with tiles
      const int m_e = sh_tiles[lo + 1] - sh_tiles[lo];
      long long rest = target - (long long)sh_cost[lo] * n_ct;
      const int ct = c_e ? (int)(rest / c_e) : 0;
      rest -= (long long)ct * c_e;
      // row tiles inside the column tile: average cost is close enough
      const int mt = c_e ? (int)(rest * m_e / c_e) : 0;
      bound = sh_tiles[lo] * n_ct + min(ct, n_ct) * m_e + min(mt, m_e);
      bound = min(bound, total_tiles);
    }
    sh_bound[g][x] = bound;
  }
  // The tile sequences (two-launch form: written by the scatter kernel's
  // workgroups instead, which are many).  The waves take the experts in turn.
  if (with_tiles) {
    for (int ee = w; ee < E; ee += 4)
      write_expert_tiles(ee, sh_nmt[ee], sh_rb[ee], sh_extra[ee], sh_rowblk[ee], sh_tiles[ee], lane,
                         n_ct_gate_up, n_ct_down, out);
  }
  __syncthreads();
  // keep every range within what the launch grid provides for (xcd_tile_cap)
  if (e < 2) {
    const int n_ct = e ? n_ct_down : n_ct_gate_up;
    const int total_tiles = tot_mt * n_ct;
    const int cap = xcd_tile_cap(total_tiles);
    int *bounds = totals + (e ? kTotBoundsDown : kTotBoundsGateUp);
    int prev = 0;
    bounds[0] = 0;
    for (int x = 1; x < kXcds; x++) {
      int bnd = sh_bound[e][x];
      bnd = max(bnd, max(prev, total_tiles - (kXcds - x) * cap));
      bnd = min(bnd, prev + cap);
      bounds[x] = bnd;
      prev = bnd;
    }
    bounds[kXcds] = total_tiles;
  }
  *ex_count_out = ex_count;
  if (tot_count_out) *tot_count_out = tot_count;
  return ex_pad;
}

// The row-tile plan (see build_plan): an expert with M rows has ceil(M / 32) row
// blocks, cut into n_mt = ceil(row blocks / 8) tiles as evenly as they go: the
// first `extra` tiles are rb + 1 row blocks high, the others rb.  Its segment in
// the padded row space is its row blocks and no more, so an expert pads to at
// most 31 rows.  The tile sequence of either GEMM (n_ct column tiles per row
// tile) is cut into the 8 ranges of the XCDs by estimated cost: a tile of r row
// blocks costs kCostPerTile + kCostPerRowBlock * r.

// Ranks inside one wave: for each of the lane's kTopK expert ids, how many of
// the wave's assignments to the same expert come before it in (lane, slot)
// order, and how many there are in all.  Instead of a loop over the experts
// (kTopK ballots each), the ids are compared bit plane by bit plane: one ballot
// per slot and bit of the id, then a lane's id selects plane or complement and
// the AND over the planes is the mask of the lanes that hold the same id in
// that slot.  The work no longer grows with the number of experts (4 x faster
// at 128).  Ids < 0 match nothing; their results are not used.
template <int NBITS>
__device__ __forceinline__ void wave_ranks(const int (&id)[kTopK], int lane, int (&rank)[kTopK],
                                           int (&total)[kTopK]) {
  unsigned long long valid[kTopK], plane[kTopK][NBITS];
#pragma unroll
  for (int k = 0; k < kTopK; k++) {
    valid[k] = __ballot(id[k] >= 0);
#pragma unroll
    for (int b = 0; b < NBITS; b++) plane[k][b] = __ballot(id[k] >= 0 && ((id[k] >> b) & 1));
  }
  const unsigned long long me = 1ull << lane;
  const unsigned long long lt = me - 1ull;
#pragma unroll
  for (int k = 0; k < kTopK; k++) {
    int r = 0, n = 0;
#pragma unroll
    for (int k2 = 0; k2 < kTopK; k2++) {
      unsigned long long m = valid[k2];
#pragma unroll
      for (int b = 0; b < NBITS; b++) m &= ((id[k] >> b) & 1) ? plane[k2][b] : ~plane[k2][b];
      n += __popcll(m);
      r += __popcll(m & lt);             // lower lanes, any slot
      if (k2 < k) r += (m & me) ? 1 : 0;  // this lane, lower slots
    }
    rank[k] = r;
    total[k] = n;
  }
}

__device__ __forceinline__ void wave_ranks_for(int E, const int (&id)[kTopK], int lane, int (&rank)[kTopK],
                                               int (&total)[kTopK]) {
  if (E <= 32) wave_ranks<5>(id, lane, rank, total);
  else if (E <= 128) wave_ranks<7>(id, lane, rank, total);
  else wave_ranks<8>(id, lane, rank, total);
}

// Pass 2: the plan and the stable permutation in one launch.  Every workgroup
// adds up the per-workgroup counts of pass 1 itself (at most a few dozen loads
// per expert): the experts' totals, from which it derives offsets and padded
// first rows exactly as workgroup 0 does, and the counts of the workgroups
// before it, its own base inside every expert.  Workgroup 0 also stores the
// plan for the GEMMs; a one-workgroup kernel between the passes did that before
// and cost a launch more than the repeated sums cost here.
// Rank of an assignment inside its expert = (assignments of lower workgroups)
// + (lower waves of this workgroup) + (lower lanes of this wave) + (lower slots
// of this token), all for the same expert.
__global__ __launch_bounds__(kDispThreads) void dispatch_scatter_kernel(
    const int *__restrict__ topk_i, const int *__restrict__ pos, int T, int E,
    const int *__restrict__ blk_counts, int n_blk, int *__restrict__ perm, int *__restrict__ rowmap,
    int *__restrict__ inv, int n_ct_gate_up, int n_ct_down, PlanOut plan) {
  __shared__ int wave_cnt[kDispThreads / 64][256];
  __shared__ int sh_base[256], sh_off[256], sh_row0[256];
  __shared__ ExpertInfo sh_info[256];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = tid >> 6;
  // the token's ids first: their loads run while the counts are added up
  const int t = blockIdx.x * kDispThreads + tid;
  int id[kTopK] = {-1, -1, -1, -1};
  if (t < T && !(pos && pos[t] < 0)) {
    const int4 ids = *reinterpret_cast<const int4 *>(topk_i + (size_t)t * kTopK);
    id[0] = ids.x; id[1] = ids.y; id[2] = ids.z; id[3] = ids.w;
#pragma unroll
    for (int k = 0; k < kTopK; k++)
      if (id[k] >= E) id[k] = -1;
  }
  int count = 0, base = 0;
  if (tid < E) {
    for (int b0 = 0; b0 < n_blk; b0 += 16) {  // 16 independent loads at a time
      int c[16];
#pragma unroll
      for (int i = 0; i < 16; i++) c[i] = b0 + i < n_blk ? blk_counts[(size_t)(b0 + i) * E + tid] : 0;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        if (b0 + i < (int)blockIdx.x) base += c[i];
        count += c[i];
      }
    }
  }
  int ex_count;
  ExpertInfo inf;
  const int row0 = build_plan(count, E, n_ct_gate_up, n_ct_down, plan, /*with_tiles=*/false, &ex_count, nullptr,
                              /*write_global=*/blockIdx.x == 0, &inf);
  sh_base[tid] = base;
  sh_off[tid] = ex_count;
  sh_row0[tid] = row0;
  sh_info[tid] = inf;
  for (int e = tid; e < (kDispThreads / 64) * 256; e += kDispThreads) (&wave_cnt[0][0])[e] = 0;
  int rank[kTopK], total[kTopK];
  wave_ranks_for(E, id, lane, rank, total);
  __syncthreads();
  // The tile sequences of the GEMMs: the waves of all workgroups take the
  // experts in turn.
  for (int ee = blockIdx.x * (kDispThreads / 64) + w; ee < E; ee += gridDim.x * (kDispThreads / 64)) {
    const ExpertInfo f = sh_info[ee];
    write_expert_tiles(ee, f.n_mt, f.rb, f.extra, f.row0 / kRowBlock, f.tile_base, lane, n_ct_gate_up,
                       n_ct_down, plan);
  }
#pragma unroll
  for (int k = 0; k < kTopK; k++)
    if (id[k] >= 0) wave_cnt[w][id[k]] = total[k];  // the same value from every lane that holds the id
  __syncthreads();
  if (t >= T) return;
  int out_inv[kTopK];
#pragma unroll
  for (int k = 0; k < kTopK; k++) {
    const int e = id[k];
    const int a = t * kTopK + k;
    if (e < 0) { out_inv[k] = -1; continue; }
    int r = sh_base[e] + rank[k];
    for (int ww = 0; ww < w; ww++) r += wave_cnt[ww][e];
    const int prow = sh_row0[e] + r;
    perm[sh_off[e] + r] = a;
    rowmap[prow] = a;
    out_inv[k] = prow;
  }
  *reinterpret_cast<int4 *>(inv + (size_t)t * kTopK) =
      make_int4(out_inv[0], out_inv[1], out_inv[2], out_inv[3]);
}

// Both passes in one workgroup for batches of at most kSmallRounds x 256 tokens:
// the rounds of 256 tokens play the part of the workgroups of the two-kernel
// form (round r's assignments come after those of the rounds before it), so
// the result is the same, bit for bit.
constexpr int kSmallRounds = 1;

__global__ __launch_bounds__(kDispThreads) void dispatch_small_kernel(
    const int *__restrict__ topk_i, const int *__restrict__ pos, int T, int E, int n_ct_gate_up,
    int n_ct_down, PlanOut out, int *__restrict__ perm, int *__restrict__ rowmap,
    int *__restrict__ inv) {
  __shared__ int hist[kSmallRounds][256];  // per round and expert: count, then exclusive base
  __shared__ int sh_off[256], sh_row0[256];
  __shared__ int wave_cnt[kDispThreads / 64][256];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = tid >> 6;
  const int n_round = (T + kDispThreads - 1) / kDispThreads;
#pragma unroll
  for (int r = 0; r < kSmallRounds; r++) hist[r][tid] = 0;
  __syncthreads();
  int id[kSmallRounds][kTopK];
#pragma unroll
  for (int r = 0; r < kSmallRounds; r++) {
    const int t = r * kDispThreads + tid;
#pragma unroll
    for (int k = 0; k < kTopK; k++) id[r][k] = -1;
    if (r < n_round && t < T && !(pos && pos[t] < 0)) {
      const int4 ids = *reinterpret_cast<const int4 *>(topk_i + (size_t)t * kTopK);
      id[r][0] = ids.x; id[r][1] = ids.y; id[r][2] = ids.z; id[r][3] = ids.w;
#pragma unroll
      for (int k = 0; k < kTopK; k++) {
        if (id[r][k] < 0 || id[r][k] >= E) id[r][k] = -1;
        if (id[r][k] >= 0) atomicAdd(&hist[r][id[r][k]], 1);
      }
    }
  }
  __syncthreads();
  // expert tid: counts of the rounds -> exclusive bases, total -> plan
  int count = 0;
#pragma unroll
  for (int r = 0; r < kSmallRounds; r++) {
    const int c = hist[r][tid];
    hist[r][tid] = count;
    count += c;
  }
  int ex_count, tot_count;
  const int row0 = build_plan(tid < E ? count : 0, E, n_ct_gate_up, n_ct_down, out, /*with_tiles=*/true, &ex_count, &tot_count);
  sh_off[tid] = ex_count;
  sh_row0[tid] = row0;
  // -1 where the scatter below writes nothing: the padding rows of the experts
  // and the tail of perm that inactive rows and invalid ids leave unused
  if (tid < E) {
    const int end = row0 + (count + kRowBlock - 1) / kRowBlock * kRowBlock;
    for (int i = row0 + count; i < end; i++) rowmap[i] = -1;
  }
  for (int i = tot_count + tid; i < T * kTopK; i += kDispThreads) perm[i] = -1;
  __syncthreads();
  // stable ranks, as dispatch_scatter_kernel
#pragma unroll
  for (int r = 0; r < kSmallRounds; r++) {
    if (r >= n_round) break;
    for (int e = tid; e < (kDispThreads / 64) * 256; e += kDispThreads) (&wave_cnt[0][0])[e] = 0;
    int rank[kTopK], total[kTopK];
    wave_ranks_for(E, id[r], lane, rank, total);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kTopK; k++)
      if (id[r][k] >= 0) wave_cnt[w][id[r][k]] = total[k];
    __syncthreads();
    const int t = r * kDispThreads + tid;
    if (t < T) {
      int out_inv[kTopK];
#pragma unroll
      for (int k = 0; k < kTopK; k++) {
        const int e = id[r][k];
        if (e < 0) { out_inv[k] = -1; continue; }
        int rk = hist[r][e] + rank[k];
        for (int ww = 0; ww < w; ww++) rk += wave_cnt[ww][e];
        const int prow = sh_row0[e] + rk;
        perm[sh_off[e] + rk] = t * kTopK + k;
        rowmap[prow] = t * kTopK + k;
        out_inv[k] = prow;
      }
      *reinterpret_cast<int4 *>(inv + (size_t)t * kTopK) =
          make_int4(out_inv[0], out_inv[1], out_inv[2], out_inv[3]);
    }
    __syncthreads();  // wave_cnt is reused by the next round
  }
}

// out[t,:] (+)= sum_k topk_v[t,k] * y[inv[t,k],:], slots added in order 0..3
// (descending router score, as reduce_mlp2_slots_kernel does,
// utility/utility.cpp:701-726).  Every token owns its K rows of y, so there
// are no atomics.
//
// RESID: instead of writing the fp32 sum, adds it to the bf16 residual stream
// in place, x = bf16(float(x) + sum) (residual_add_batch_kernel,
// utility/utility.cpp:158-173; call getp_run.cpp:846-852); inactive rows are
// left alone.
//
// DIRECT: there was no dispatch pass (see DirectIds).  The row of assignment
// (t, k) is its expert's slot plus the number of lower assignments of the batch
// with the same expert, which the workgroup's 256 threads count with a ballot.
// SPLIT: the down GEMM summed its reduction in two parts (down_k_split); the
// second part's rows lie part_stride floats behind the first's and are added to
// them before the weighting.
template <bool RESID, bool DIRECT, bool SPLIT>
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y,
                                                     const int *__restrict__ inv,
                                                     const float *__restrict__ topk_v,
                                                     const int *__restrict__ pos, void *outp, int H,
                                                     int ldy, int accumulate, DirectIds ids,
                                                     size_t part_stride) {
  const int t = blockIdx.x;
  const bool active = !(pos && pos[t] < 0);
  if (!active && (accumulate || RESID)) return;
  int p[kTopK] = {-1, -1, -1, -1};
  float w[kTopK] = {0.f, 0.f, 0.f, 0.f};
  if (DIRECT) {
    __shared__ int lower[256 / 64][kTopK];
    const int tid = threadIdx.x;
    const int mine = direct_expert_of(ids, tid);
    int e[kTopK];
#pragma unroll
    for (int k = 0; k < kTopK; k++) {
      e[k] = direct_expert_of(ids, t * kTopK + k);
      const unsigned long long bal = __ballot(e[k] >= 0 && mine == e[k] && tid < t * kTopK + k);
      if ((tid & 63) == 0) lower[tid >> 6][k] = __popcll(bal);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kTopK; k++) {
      const int r = lower[0][k] + lower[1][k] + lower[2][k] + lower[3][k];
      if (e[k] >= 0 && r < kDirectSlotRows) p[k] = e[k] * kDirectSlotRows + r;
    }
    if (active) {
      const float4 wv = *reinterpret_cast<const float4 *>(topk_v + (size_t)t * kTopK);
      w[0] = wv.x; w[1] = wv.y; w[2] = wv.z; w[3] = wv.w;
    }
  } else if (active) {
    const int4 pi = *reinterpret_cast<const int4 *>(inv + (size_t)t * kTopK);
    const float4 wv = *reinterpret_cast<const float4 *>(topk_v + (size_t)t * kTopK);
    p[0] = pi.x; p[1] = pi.y; p[2] = pi.z; p[3] = pi.w;
    w[0] = wv.x; w[1] = wv.y; w[2] = wv.z; w[3] = wv.w;
  }
  float4 *o = reinterpret_cast<float4 *>(reinterpret_cast<float *>(outp) + (size_t)t * H);
  uint2 *xr = reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(outp) + (size_t)t * H);
  for (int c = threadIdx.x; c < H / 4; c += 256) {
    float4 s = (!RESID && accumulate) ? o[c] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int k = 0; k < kTopK; k++) {
      if (p[k] >= 0) {
        float4 v = reinterpret_cast<const float4 *>(y + (size_t)p[k] * ldy)[c];
        if (SPLIT) {
          const float4 v2 = reinterpret_cast<const float4 *>(y + part_stride + (size_t)p[k] * ldy)[c];
          v.x += v2.x; v.y += v2.y; v.z += v2.z; v.w += v2.w;
        }
        s.x += w[k] * v.x; s.y += w[k] * v.y; s.z += w[k] * v.z; s.w += w[k] * v.w;
      }
    }
    if (RESID) {
      const uint2 xv = xr[c];
      const float r0 = __uint_as_float(xv.x << 16) + s.x, r1 = __uint_as_float(xv.x & 0xffff0000u) + s.y;
      const float r2 = __uint_as_float(xv.y << 16) + s.z, r3 = __uint_as_float(xv.y & 0xffff0000u) + s.w;
      xr[c] = make_uint2(f32_to_bf16_rne(r0) | ((uint32_t)f32_to_bf16_rne(r1) << 16),
                         f32_to_bf16_rne(r2) | ((uint32_t)f32_to_bf16_rne(r3) << 16));
    } else {
      o[c] = s;
    }
  }
}

hipError_t launch_dispatch(const int *topk_i, const int *pos, int T, int E, int n_ct_gate_up,
                           int n_ct_down, const DispatchBuffers &d, hipStream_t s) {
  const int n_blk = (T + kDispThreads - 1) / kDispThreads;
  // Rows of the padded space this batch can reach: every expert rounds its
  // rows up to a multiple of 32.
  const long long A = (long long)T * kTopK;
  const long long reach = A + (long long)kTileGran * E;
  const int fill_rows = (int)(reach < d.a_pad_cap ? reach : d.a_pad_cap);
  PlanOut plan;
  plan.offsets = d.offsets;
  plan.info = d.info;
  plan.totals = d.totals;
  plan.tiles_gate_up = d.tiles_gate_up;
  plan.tiles_down = d.tiles_down;
  plan.tile_cap_gate_up = d.tile_cap_gate_up;
  plan.tile_cap_down = d.tile_cap_down;
  if (n_blk <= kSmallRounds) {
    // small batches: one workgroup does both passes, one launch fewer
    dispatch_small_kernel<<<1, kDispThreads, 0, s>>>(topk_i, pos, T, E, n_ct_gate_up, n_ct_down, plan,
                                                     d.perm, d.rowmap, d.inv);
    return hipGetLastError();
  }
  dispatch_count_kernel<<<n_blk, kDispThreads, 0, s>>>(topk_i, pos, T, E, d.blk_counts, d.rowmap,
                                                       fill_rows, d.perm);
  dispatch_scatter_kernel<<<n_blk, kDispThreads, 0, s>>>(topk_i, pos, T, E, d.blk_counts, n_blk, d.perm,
                                                         d.rowmap, d.inv, n_ct_gate_up, n_ct_down, plan);
  return hipGetLastError();
}

template <bool RESID>
static hipError_t launch_combine_any(const float *y, int ldy, int y_parts, size_t part_stride, const int *inv,
                                     const float *topk_v, const int *pos, void *out, int T, int H,
                                     int accumulate, const DirectIds &direct, hipStream_t s) {
  static_assert(kSmallBatchKSplit == 2, "the combine adds two parts");
  if (y_parts != 1 && y_parts != kSmallBatchKSplit) return hipErrorInvalidValue;
  const bool split = y_parts == 2;
#define MOE_COMBINE(DIRECT, SPLIT)                                                                             \
  combine_kernel<RESID, DIRECT, SPLIT><<<T, 256, 0, s>>>(y, inv, topk_v, pos, out, H, ldy, accumulate, direct, \
                                                         part_stride)
  if (direct.topk_i) {
    if (split) MOE_COMBINE(true, true); else MOE_COMBINE(true, false);
  } else {
    if (split) MOE_COMBINE(false, true); else MOE_COMBINE(false, false);
  }
#undef MOE_COMBINE
  return hipGetLastError();
}

hipError_t launch_combine(const float *y, int ldy, int y_parts, size_t part_stride, const int *inv,
                          const float *topk_v, const int *pos, float *out, int T, int H, int accumulate,
                          const DirectIds &direct, hipStream_t s) {
  return launch_combine_any<false>(y, ldy, y_parts, part_stride, inv, topk_v, pos, out, T, H, accumulate, direct,
                                   s);
}

hipError_t launch_combine_residual(const float *y, int ldy, int y_parts, size_t part_stride, const int *inv,
                                   const float *topk_v, const int *pos, uint16_t *x, int T, int H,
                                   const DirectIds &direct, hipStream_t s) {
  return launch_combine_any<true>(y, ldy, y_parts, part_stride, inv, topk_v, pos, x, T, H, 0, direct, s);
}

}  // namespace moe

// ---- dispatch for callers that cannot allocate ----
//
// moe_dispatch_static runs the same kernels as moe_dispatch, but needs no
// handle and calls no allocating routine: the buffers the kernels use beyond
// the caller's inputs and outputs (per-workgroup counts, the padded row map,
// the inverse map, the per-expert records and the plan's totals) live in one
// file-scope device array.  Every GPU the library runs on holds that array
// until the process ends; every call on a GPU shares it, so calls that overlap
// on one GPU (two streams, two threads) race.  The kernels rewrite everything
// they later read, so nothing of an earlier call survives into the next.
namespace moe {
namespace {

constexpr int kStaticMaxTokens = MOE_DISPATCH_STATIC_MAX_TOKENS;
constexpr int kStaticMaxExperts = MOE_DISPATCH_STATIC_MAX_EXPERTS;
constexpr size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
constexpr size_t kStaticBlkCounts = 0;
constexpr size_t kStaticRowmap =
    kStaticBlkCounts + align256(sizeof(int) * ((kStaticMaxTokens + kDispThreads - 1) / kDispThreads) * kStaticMaxExperts);
constexpr int kStaticPadRows = kStaticMaxTokens * kTopK + kTileGran * kStaticMaxExperts;
constexpr size_t kStaticInv = kStaticRowmap + align256(sizeof(int) * kStaticPadRows);
constexpr size_t kStaticInfo = kStaticInv + align256(sizeof(int) * kStaticMaxTokens * kTopK);
constexpr size_t kStaticTotals = kStaticInfo + align256(sizeof(ExpertInfo) * kStaticMaxExperts);
constexpr size_t kStaticBytes = kStaticTotals + align256(sizeof(int) * kTotInts);

static __device__ __align__(256) unsigned char scratch[kStaticBytes];

// Device address of this GPU's copy of `scratch`: looked up once per device
// (each GPU holds its own copy at its own address), never taken from the
// array's name, which on the host is only a stand-in for the symbol.
constexpr int kMaxDevices = 64;
unsigned char *g_scratch_ptr[kMaxDevices];  // written once per device, then only read

hipError_t static_scratch(unsigned char **out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  unsigned char *p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);  // the same value from every thread
  }
  *out = p;
  return hipSuccess;
}

}  // namespace
}  // namespace moe

extern "C" int moe_dispatch_static(const int *topk_i, const int *pos, int n_tokens, int n_experts,
                                   int *offsets, int *perm, void *stream) {
  using namespace moe;
  if (n_tokens < 0) return set_error(MOE_ERR_BAD_ARG, "n_tokens %d is negative", n_tokens);
  if (n_tokens > kStaticMaxTokens)
    return set_error(MOE_ERR_CAPACITY, "moe_dispatch_static: n_tokens %d exceeds its fixed maximum of %d",
                     n_tokens, kStaticMaxTokens);
  if (n_experts < 1 || n_experts > kStaticMaxExperts)
    return set_error(MOE_ERR_CAPACITY, "moe_dispatch_static: n_experts %d outside [1,%d]", n_experts,
                     kStaticMaxExperts);
  if (!offsets || (n_tokens > 0 && (!topk_i || !perm)))
    return set_error(MOE_ERR_BAD_ARG, "null device pointer");
  unsigned char *base = nullptr;
  const hipError_t e = static_scratch(&base);
  if (e != hipSuccess)
    return set_error(MOE_ERR_HIP, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
  DispatchBuffers d{};
  d.blk_counts = reinterpret_cast<int *>(base + kStaticBlkCounts);
  d.rowmap = reinterpret_cast<int *>(base + kStaticRowmap);
  d.inv = reinterpret_cast<int *>(base + kStaticInv);
  d.info = reinterpret_cast<ExpertInfo *>(base + kStaticInfo);
  d.totals = reinterpret_cast<int *>(base + kStaticTotals);
  d.offsets = offsets;
  d.perm = perm;
  d.a_pad_cap = kStaticPadRows;
  // no GEMM follows: with no column tiles the plan kernel writes no tile tables
  d.tiles_gate_up = d.tiles_down = nullptr;
  d.tile_cap_gate_up = d.tile_cap_down = 0;
  const hipError_t el = launch_dispatch(topk_i, pos, n_tokens, n_experts, 0, 0, d, static_cast<hipStream_t>(stream));
  if (el != hipSuccess)
    return set_error(MOE_ERR_HIP, "dispatch launch failed: %s", hipGetErrorString(el));
  return MOE_OK;
}
