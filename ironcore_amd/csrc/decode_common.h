// Pieces shared by the decode kernels: kernel parameters, the balanced
// split-K bookkeeping (every wave finds its own share of the batch-wide tile
// sequence) and the per-window gather of tile addresses.
#pragma once

#include "ic_device.h"
#include "ic_internal.h"

namespace ic {
namespace decode {

struct DecodeKP {
  const char *q;
  const char *k_pool;
  const char *v_pool;
  const int32_t *block_tables;
  const int32_t *context_lens;
  char *out;
  int32_t *cum_blocks;  // [n_seqs + 1] exclusive prefix sum of per-sequence block counts
  float *part_ml;       // [n_partials, GT, 2]
  float *part_acc;      // [n_partials, GT, hd]
  int64_t q_stride_seq;    // elements
  int64_t out_stride_seq;  // elements
  int64_t stride_block;    // elements
  int64_t stride_head;
  int64_t stride_token;
  int64_t bt_stride;
  int64_t num_blocks;
  int n_seqs;
  int hn;
  int group;        // query heads per KV head
  int nsub;         // query sub-groups per KV head (ceil(group / GT))
  int gt;           // matrix columns per pair = query heads per sub-group, times the
                    // cohort size with cohorts (the stride of the partial arrays)
  int pairs_per_seq;  // gn * nsub
  int max_ctx;
  int n_waves;      // waves in the main kernel's grid
  int max_waves;    // most waves the partial arrays have slots for (host side: caps the grid)
  int min_chunk;    // smallest chunk, in tiles
  int tiles_per_block;  // 16-token tiles in one pool block (1 for block_size 16)
  float scale_log2e;
  // Shared-prefix cohorts (matrix-core kernel only).  cohort_size consecutive
  // sequences form a cohort whose first cohort_shared[c] pool blocks are the
  // same physical blocks.  The kernel then works in two phases, each with its
  // own balanced split of its own tile sequence:
  //   own phase     rows = sequences, each from its cohort's shared tiles on;
  //                 a share belongs to one wave (as without cohorts);
  //   shared phase  rows = cohorts, the shared tiles; a share belongs to a UNIT
  //                 of 2^unit_shift neighbouring waves of one workgroup, which
  //                 walk the same tiles at the same time, wave j of the unit
  //                 with members j*spw .. j*spw+spw-1 as its matrix columns: the
  //                 tile comes from HBM once and from the cache for the others.
  const int32_t *cohort_shared;  // [n_cohorts] pool blocks, or nullptr
  int32_t *cum_shared;           // [n_cohorts + 1] prefix sums of the shared phase's rows
  int64_t shared_slot0;          // first partial slot of the shared phase
  int cohort_size;               // S >= 1
  int n_cohorts;
  int spw;
  int unit_shift;
  // Key mask (vector-ALU kernel only; nullptr = every key of the context is visible): byte
  // (sequence i, query head h, key j) at key_mask[i*key_mask_stride_seq + h*key_mask_stride_head + j],
  // nonzero = visible.
  const uint8_t *key_mask;
  int64_t key_mask_stride_seq;
  int64_t key_mask_stride_head;
};

constexpr float kNegInf = -__builtin_huge_valf();
// Score (log2 units) of a key the mask hides: the reference fills hidden scores with the FINITE
// minimum of the element type (attention.py:66,115-117), so beside a visible key a hidden one
// weighs nothing, while a row with no visible key averages V over its whole context.
constexpr float kHiddenLog2 = -0x1p100f;

__device__ __forceinline__ int seq_blocks(const DecodeKP &p, int seq, int bs) {
  int ctx = p.context_lens[seq];
  ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
  return ctx > 0 ? (ctx + bs - 1) / bs : 0;
}

// Tiles of cohort c that are streamed once for all members: the caller's
// count of aliased blocks, cut down to whole tiles every member's context
// covers (so a shared tile never needs a mask).
__device__ __forceinline__ int cohort_shared_tiles(const DecodeKP &p, int c) {
  int sh = p.cohort_shared[c] * p.tiles_per_block;
  for (int u = 0; u < p.cohort_size; ++u) {
    const int s = c * p.cohort_size + u;
    if (s >= p.n_seqs) break;
    int ctx = p.context_lens[s];
    ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
    const int whole = ctx > 0 ? ctx / 16 : 0;
    sh = sh < whole ? sh : whole;
  }
  return sh > 0 ? sh : 0;
}

// A row of the work layout: which sequence's block table it walks, its
// first tile in that sequence and how many tiles it has.
struct RowSpan {
  int tseq;   // sequence whose block-table row addresses the tiles
  int first;  // first tile (of the sequence) in this row
  int tiles;
};

template <int BS>
__device__ __forceinline__ RowSpan row_span(const DecodeKP &p, int shared, int row) {
  if (p.cohort_size == 1) return RowSpan{row, 0, seq_blocks(p, row, BS)};
  if (shared) return RowSpan{row * p.cohort_size, 0, cohort_shared_tiles(p, row)};
  const int sh = cohort_shared_tiles(p, row / p.cohort_size);
  return RowSpan{row, sh, seq_blocks(p, row, BS) - sh};
}

// Rows and shares of a phase.
__device__ __forceinline__ int phase_rows(const DecodeKP &p, int shared) { return shared ? p.n_cohorts : p.n_seqs; }
__device__ __forceinline__ int phase_units(const DecodeKP &p, int shared) {
  return shared ? p.n_waves >> p.unit_shift : p.n_waves;
}

// Tiles per share: equal shares of the N tiles, never below min_chunk.
__device__ __forceinline__ int64_t chunk_tiles(const DecodeKP &p, int64_t n_tiles, int units) {
  int64_t c = (n_tiles + units - 1) / units;
  return c < p.min_chunk ? p.min_chunk : c;
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int up = __shfl_up(v, off, kWave);
    v += lane >= off ? up : 0;
  }
  return v;
}

// Position in the batch-wide tile sequence: tile `blk` of pair (row, pair)
// whose row has `nb` tiles.  Wave-uniform.
struct TileCursor {
  int seq;    // row (= sequence when there are no cohorts)
  int pair;
  int blk;
  int nb;
  int tseq;   // block-table row of this row's tiles
  int first;  // tile of that sequence the row starts at
};

__device__ __forceinline__ void set_row(TileCursor &c, int row, const RowSpan &r) {
  c.seq = row;
  c.nb = __builtin_amdgcn_readfirstlane(r.tiles);  // wave-uniform: keep it scalar
  c.tseq = __builtin_amdgcn_readfirstlane(r.tseq);
  c.first = __builtin_amdgcn_readfirstlane(r.first);
}

// Where a phase's rows come from.  GlobalRows derives a row from the
// caller's arrays every time it is asked (a few dependent loads, and one per
// cohort member); PlannedRows reads the prefix sums a workgroup has laid out
// in LDS once (build_plan below).
template <int BS>
struct GlobalRows {
  const DecodeKP &p;
  int shared;
  __device__ __forceinline__ int n_rows() const { return phase_rows(p, shared); }
  __device__ __forceinline__ RowSpan span(int row) const { return row_span<BS>(p, shared, row); }
};

struct PlannedRows {
  const int *cum;     // LDS: [n + 1] exclusive prefix sums of the phase's row tile counts
  const int *eff_sh;  // LDS: [n_cohorts] shared tiles per cohort (cohorts only)
  int n;
  int cohort_size;
  int shared;
  __device__ __forceinline__ int n_rows() const { return n; }
  __device__ __forceinline__ RowSpan span(int row) const {
    const int tiles = cum[row + 1] - cum[row];
    if (cohort_size == 1) return RowSpan{row, 0, tiles};
    if (shared) return RowSpan{row * cohort_size, 0, tiles};
    return RowSpan{row, eff_sh[row / cohort_size], tiles};
  }
};

template <class Rows>
__device__ __forceinline__ void next_pair(const DecodeKP &p, const Rows &rows, TileCursor &c) {
  c.blk = 0;
  if (++c.pair == p.pairs_per_seq) {
    c.pair = 0;
    const int n_rows = rows.n_rows();
    do {
      ++c.seq;
      if (c.seq >= n_rows) {  // past the last tile: never dereferenced
        c.seq = n_rows;
        c.nb = 0x7fffffff;
        return;
      }
      set_row(c, c.seq, rows.span(c.seq));
    } while (c.nb == 0);
  }
}

// Workgroups are dealt to the 8 XCDs round-robin by launch index.  Shares of
// the tile sequence are handed out XCD-major instead, so that neighbouring
// shares (sequences that may alias the same prefix blocks, and the query
// sub-groups of one KV head) run on one XCD at the same time and meet in its
// L2 instead of each fetching the blocks from HBM.
__device__ __forceinline__ int xcd_major_workgroup() {
  int wg = blockIdx.x;
  if ((gridDim.x & 7) == 0) wg = (wg & 7) * (gridDim.x >> 3) + (wg >> 3);
  return wg;
}

// Share `wid` of a phase: [t0, t0 + left) of its tile sequence and the
// cursor of its first tile.  Every wave prefix-sums the per-row tile counts
// itself (kRowsPerLane consecutive rows per lane and step, their loads in
// flight together): first for the total, which fixes the chunk size, then
// again to find the row that holds its first tile.  Share 0 also leaves the
// prefix sums in the workspace for the reduce kernel.  Returns false when the
// wave has no tiles.
constexpr int kRowsPerLane = 4;

template <int BS>
__device__ __forceinline__ bool locate_chunk(const DecodeKP &p, int lane, int shared, int64_t wid,
                                             int64_t &left, TileCursor &c) {
  constexpr int RPS = kWave * kRowsPerLane;  // rows per step
  const int n_rows = phase_rows(p, shared);
  int32_t *cum_out = shared ? p.cum_shared : p.cum_blocks;
  int64_t total = 0;
  for (int base = 0; base < n_rows; base += RPS) {
    int cnt[kRowsPerLane];
#pragma unroll
    for (int k = 0; k < kRowsPerLane; ++k) {
      const int r = base + lane * kRowsPerLane + k;
      cnt[k] = r < n_rows ? row_span<BS>(p, shared, r).tiles : 0;
    }
    int mine = 0;
#pragma unroll
    for (int k = 0; k < kRowsPerLane; ++k) mine += cnt[k];
    const int incl = wave_inclusive_scan(mine, lane);
    if (wid == 0) {
      int run = (int)total + incl - mine;
#pragma unroll
      for (int k = 0; k < kRowsPerLane; ++k) {
        const int r = base + lane * kRowsPerLane + k;
        run += cnt[k];
        if (r < n_rows) cum_out[r + 1] = run;
      }
    }
    total += __builtin_amdgcn_readlane(incl, kWave - 1);
  }
  if (wid == 0 && lane == 0) cum_out[0] = 0;
  const int64_t n_tiles = total * p.pairs_per_seq;
  const int64_t chunk = chunk_tiles(p, n_tiles, phase_units(p, shared));
  const int64_t t0 = wid * chunk;
  if (t0 >= n_tiles) return false;
  left = (t0 + chunk < n_tiles ? t0 + chunk : n_tiles) - t0;

  int64_t before = 0;  // tiles of the rows scanned so far
  int row = n_rows;
  int cum = 0;
  for (int base = 0; base < n_rows; base += RPS) {
    int cnt[kRowsPerLane];
#pragma unroll
    for (int k = 0; k < kRowsPerLane; ++k) {
      const int r = base + lane * kRowsPerLane + k;
      cnt[k] = r < n_rows ? row_span<BS>(p, shared, r).tiles : 0;
    }
    int mine = 0;
#pragma unroll
    for (int k = 0; k < kRowsPerLane; ++k) mine += cnt[k];
    const int incl = wave_inclusive_scan(mine, lane);
    // first lane whose rows end after t0
    const uint64_t hit = __ballot((before + incl) * p.pairs_per_seq > t0);
    if (hit != 0) {
      const int ln = __builtin_ctzll(hit);
      int run = (int)before + __builtin_amdgcn_readlane(incl - mine, ln);
      int found = -1, found_cum = 0;
#pragma unroll
      for (int k = 0; k < kRowsPerLane; ++k) {
        const int n = __builtin_amdgcn_readlane(cnt[k], ln);
        if (found < 0 && (int64_t)(run + n) * p.pairs_per_seq > t0) {
          found = k;
          found_cum = run;
        }
        run += n;
      }
      row = base + ln * kRowsPerLane + found;
      cum = found_cum;
      break;
    }
    before += __builtin_amdgcn_readlane(incl, kWave - 1);
  }
  row = __builtin_amdgcn_readfirstlane(row);
  set_row(c, row, row_span<BS>(p, shared, row));
  const int64_t r = t0 - (int64_t)cum * p.pairs_per_seq;
  c.pair = (int)(r / c.nb);
  c.blk = (int)(r - (int64_t)c.pair * c.nb);
  return true;
}

// ---- row bookkeeping in LDS ---------------------------------------------------
// Every wave needs the prefix sums of the rows' tile counts to find its share.
// Scanning the rows per wave (locate_chunk) costs a few dependent round trips
// per 256 rows and, with cohorts, one load per member and row; a workgroup can
// instead lay the prefix sums out in LDS once, all its threads sharing the
// loads, and its waves then search LDS.  Layout (ints): eff_sh [C] | cum_sh
// [C + 1] | cum_own [R + 1] | scratch [kPlanScratch].
constexpr int kPlanScratch = 16;
constexpr int kPlanMaxInts = 12000;  // 48 KB of LDS per workgroup at most

struct PlanLds {
  int *eff_sh;
  int *cum_sh;
  int *cum_own;
  int *scratch;
};

__host__ __device__ inline size_t plan_ints(int n_seqs, int n_cohorts) {
  return (size_t)n_cohorts + ((size_t)n_cohorts + 1) + ((size_t)n_seqs + 1) + kPlanScratch;
}

// The tile ring of the cooperative shared phase follows the plan, 16-byte aligned.
__host__ __device__ inline size_t ring_offset_ints(int n_seqs, int n_cohorts) {
  return (plan_ints(n_seqs, n_cohorts) + 3) & ~(size_t)3;
}
// LDS behind the plan: a K tile per wave for staging (16 rows of hd 16-bit
// elements, padded by 16 bytes each) and, with `coop`, a ring of one such K
// tile and one V tile per wave of the workgroup.
__host__ __device__ constexpr size_t tiles_lds_bytes(int hd, int waves, bool coop) {
  return (size_t)waves * (16 * (hd * 2 + 16)) + (coop ? (size_t)waves * (16 * (hd * 2 + 16) + 16 * hd * 2) : 0);
}

__device__ __forceinline__ PlanLds plan_carve(int *base, const DecodeKP &p) {
  PlanLds pl;
  pl.eff_sh = base;
  pl.cum_sh = pl.eff_sh + p.n_cohorts;
  pl.cum_own = pl.cum_sh + p.n_cohorts + 1;
  pl.scratch = pl.cum_own + p.n_seqs + 1;
  return pl;
}

// out[0 .. n] = exclusive prefix sums of f(0) .. f(n-1), by all T threads of
// the workgroup (thread t takes a contiguous run of rows).  Ends with a barrier.
template <int T, class F>
__device__ __forceinline__ void block_prefix_sums(int n, F f, int *out, int *scratch) {
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int per = (n + T - 1) / T;
  const int r0 = tid * per < n ? tid * per : n;
  const int r1 = r0 + per < n ? r0 + per : n;
  int sum = 0;
  for (int r = r0; r < r1; ++r) sum += f(r);
  const int incl = wave_inclusive_scan(sum, lane);
  if (lane == kWave - 1) scratch[wave] = incl;
  __syncthreads();
  int run = incl - sum, total = 0;
#pragma unroll
  for (int w = 0; w < T / kWave; ++w) {
    const int v = scratch[w];
    run += w < wave ? v : 0;
    total += v;
  }
  for (int r = r0; r < r1; ++r) {
    out[r] = run;
    run += f(r);
  }
  if (tid == 0) out[n] = total;
  __syncthreads();
}

// Builds the plan; `publish` (one workgroup of the grid) also leaves the prefix
// sums in the workspace for the reduce kernel.
template <int BS, int T>
__device__ __forceinline__ void build_plan(const DecodeKP &p, const PlanLds &pl, bool publish) {
  const int tid = threadIdx.x;
  const bool cohorts = p.cohort_size > 1;
  if (cohorts) {
    // cohort_shared_tiles for every cohort at once: the caller's count, then the minimum over the
    // members' whole tiles, one member per thread (all context lengths in one round trip)
    for (int c = tid; c < p.n_cohorts; c += T) {
      const int sh = p.cohort_shared[c] * p.tiles_per_block;
      pl.eff_sh[c] = sh > 0 ? sh : 0;
    }
    __syncthreads();
    for (int r = tid; r < p.n_seqs; r += T) {
      int ctx = p.context_lens[r];
      ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
      atomicMin(&pl.eff_sh[r / p.cohort_size], ctx > 0 ? ctx / 16 : 0);
    }
    __syncthreads();
    block_prefix_sums<T>(p.n_cohorts, [&](int c) { return pl.eff_sh[c]; }, pl.cum_sh, pl.scratch);
    block_prefix_sums<T>(p.n_seqs, [&](int r) { return seq_blocks(p, r, BS) - pl.eff_sh[r / p.cohort_size]; },
                         pl.cum_own, pl.scratch);
  } else {
    block_prefix_sums<T>(p.n_seqs, [&](int r) { return seq_blocks(p, r, BS); }, pl.cum_own, pl.scratch);
  }
  if (publish) {
    for (int r = tid; r <= p.n_seqs; r += T) p.cum_blocks[r] = pl.cum_own[r];
    if (cohorts)
      for (int c = tid; c <= p.n_cohorts; c += T) p.cum_shared[c] = pl.cum_sh[c];
  }
}

// locate_chunk on a plan: share `wid` of `units` of the phase whose prefix
// sums are cum[0 .. n_rows].  64-way search: each round the lanes probe 64
// evenly spaced entries of the bracket.
__device__ __forceinline__ bool locate_planned(const DecodeKP &p, const PlannedRows &rows, int units, int lane,
                                               int64_t wid, int64_t &left, TileCursor &c) {
  const int n_rows = rows.n;
  const int64_t n_tiles = (int64_t)rows.cum[n_rows] * p.pairs_per_seq;
  const int64_t chunk = chunk_tiles(p, n_tiles, units);
  const int64_t t0 = wid * chunk;
  if (t0 >= n_tiles) return false;
  left = (t0 + chunk < n_tiles ? t0 + chunk : n_tiles) - t0;
  int lo = 0, hi = n_rows;  // the row is the last one in [lo, hi) whose prefix sum does not exceed t0
  while (hi - lo > 1) {
    const int step = (hi - lo + kWave - 1) / kWave;
    const int idx = lo + lane * step;
    const int v = rows.cum[idx < hi ? idx : hi];
    const uint64_t over = __ballot(idx >= hi || (int64_t)v * p.pairs_per_seq > t0);
    const int f = over != 0 ? __builtin_ctzll(over) : kWave;  // lane 0 probes lo: never over
    const int lo_new = lo + (f - 1) * step;
    hi = lo + f * step < hi ? lo + f * step : hi;
    lo = lo_new;
  }
  const int row = __builtin_amdgcn_readfirstlane(lo);
  set_row(c, row, rows.span(row));
  const int64_t r = t0 - (int64_t)rows.cum[row] * p.pairs_per_seq;
  c.pair = (int)(r / c.nb);
  c.blk = (int)(r - (int64_t)c.pair * c.nb);
  return true;
}

// Window = the next n_win (<= 64*SW) tiles of the share.  Each lane looks up
// the pool block of SW of them and keeps the tile's byte offset (the same for
// the K and the V pool); `walk` advances past the window.
template <int BS, int SW, int ES, class Rows>
__device__ __forceinline__ void gather_window(const DecodeKP &p, const Rows &rows, int lane, int n_win,
                                              TileCursor &walk, uint32_t *off_lo, uint32_t *off_hi) {
  int64_t row_idx[SW];
  int32_t kv_of[SW], sub_of[SW];
#pragma unroll
  for (int r = 0; r < SW; ++r) {
    row_idx[r] = 0;
    kv_of[r] = 0;
    sub_of[r] = 0;
  }
  for (int pos = 0; pos < n_win;) {  // wave-uniform walk over the window's segments
    const int cnt = (walk.nb - walk.blk < n_win - pos) ? walk.nb - walk.blk : n_win - pos;
    const int kvh = walk.pair / p.nsub;
    const int64_t row = (int64_t)walk.tseq * p.bt_stride;
#pragma unroll
    for (int r = 0; r < SW; ++r) {
      const int lp = r * kWave + lane;
      const bool in = lp >= pos && lp < pos + cnt;
      int tile_in_seq = walk.first + walk.blk + lp - pos;
      int sub = 0;
      if (p.tiles_per_block > 1) {  // pool blocks longer than one tile
        const int b = tile_in_seq / p.tiles_per_block;
        sub = tile_in_seq - b * p.tiles_per_block;
        tile_in_seq = b;
      }
      row_idx[r] = in ? row + tile_in_seq : row_idx[r];
      kv_of[r] = in ? kvh : kv_of[r];
      sub_of[r] = in ? sub : sub_of[r];
    }
    pos += cnt;
    walk.blk += cnt;
    if (walk.blk == walk.nb) next_pair(p, rows, walk);
  }
#pragma unroll
  for (int r = 0; r < SW; ++r) {
    int64_t phys = 0;
    if (r * kWave + lane < n_win) phys = p.block_tables[row_idx[r]];
    // A corrupt table entry must not become an out-of-pool address.
    phys = phys < 0 ? 0 : phys;
    phys = phys >= p.num_blocks ? p.num_blocks - 1 : phys;
    const int64_t off = (phys * p.stride_block + (int64_t)kv_of[r] * p.stride_head +
                         (int64_t)sub_of[r] * BS * p.stride_token) * ES;
    off_lo[r] = (uint32_t)off;
    off_hi[r] = (uint32_t)(off >> 32);
  }
}

// Byte offset of the window's i-th tile as a wave-uniform scalar (SW == 4).
__device__ __forceinline__ int64_t window_tile_offset(const uint32_t *off_lo, const uint32_t *off_hi, int i) {
  const int ln = i & (kWave - 1);
  uint32_t lo, hi;
  if (i < kWave) {
    lo = __builtin_amdgcn_readlane(off_lo[0], ln);
    hi = __builtin_amdgcn_readlane(off_hi[0], ln);
  } else if (i < 2 * kWave) {
    lo = __builtin_amdgcn_readlane(off_lo[1], ln);
    hi = __builtin_amdgcn_readlane(off_hi[1], ln);
  } else if (i < 3 * kWave) {
    lo = __builtin_amdgcn_readlane(off_lo[2], ln);
    hi = __builtin_amdgcn_readlane(off_hi[2], ln);
  } else {
    lo = __builtin_amdgcn_readlane(off_lo[3], ln);
    hi = __builtin_amdgcn_readlane(off_hi[3], ln);
  }
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

constexpr int kDecodeWavesPerWorkgroup = 4;

// Launches the matrix-core decode main kernel (paged_decode_mfma.hip) when it
// is built for this shape (16-bit dtype, hd 32, 64 or 128, kp.gt <= 16 columns);
// returns false otherwise.  Sets kp.n_waves.
bool launch_decode_mfma_main(DecodeKP &kp, int dtype, int hd, hipStream_t stream);
// Runtime occupancy queries the matrix-core launcher has made in this process.
long long decode_occupancy_queries();

}  // namespace decode
}  // namespace ic
