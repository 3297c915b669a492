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
  int gt;           // query heads per sub-group (the stride of the partial arrays)
  int pairs_per_seq;  // gn * nsub
  int max_ctx;
  int n_waves;      // waves in the main kernel's grid
  int min_chunk;    // smallest chunk, in tiles
  int tiles_per_block;  // 16-token tiles in one pool block (1 for block_size 16)
  float scale_log2e;
};

constexpr float kNegInf = -__builtin_huge_valf();

__device__ __forceinline__ int seq_blocks(const DecodeKP &p, int seq, int bs) {
  int ctx = p.context_lens[seq];
  ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
  return ctx > 0 ? (ctx + bs - 1) / bs : 0;
}

// Tiles per wave: equal shares of the N tiles, never below min_chunk.
__device__ __forceinline__ int64_t chunk_tiles(const DecodeKP &p, int64_t n_tiles) {
  int64_t c = (n_tiles + p.n_waves - 1) / p.n_waves;
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

// Position in the batch-wide tile sequence: block `blk` of pair
// (seq, pair) whose sequence has `nb` blocks.  Wave-uniform.
struct TileCursor {
  int seq;
  int pair;
  int blk;
  int nb;
};

template <int BS>
__device__ __forceinline__ void next_pair(const DecodeKP &p, TileCursor &c) {
  c.blk = 0;
  if (++c.pair == p.pairs_per_seq) {
    c.pair = 0;
    do {
      ++c.seq;
      if (c.seq >= p.n_seqs) {  // past the last tile: never dereferenced
        c.seq = p.n_seqs;
        c.nb = 0x7fffffff;
        return;
      }
      c.nb = __builtin_amdgcn_readfirstlane(seq_blocks(p, c.seq, BS));  // wave-uniform: keep it scalar
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

// This wave's share: [t0, t0 + left) of the batch-wide tile sequence and the
// cursor of its first tile.  Every wave prefix-sums the per-sequence block
// counts itself (64 sequences per step, one per lane): first for the total,
// which fixes the chunk size, then again to find the sequence that holds its
// first tile.  Wave 0 also leaves the prefix sums in the workspace for the
// reduce kernel.  Returns false when the wave has no tiles.
template <int BS>
__device__ __forceinline__ bool locate_chunk(const DecodeKP &p, int lane, int64_t wid, int64_t &left,
                                             TileCursor &c) {
  int64_t total_blocks = 0;
  for (int base = 0; base < p.n_seqs; base += kWave) {
    const int s = base + lane;
    const int mine = s < p.n_seqs ? seq_blocks(p, s, BS) : 0;
    const int incl = wave_inclusive_scan(mine, lane);
    if (wid == 0 && s < p.n_seqs) p.cum_blocks[s + 1] = (int32_t)(total_blocks + incl);
    total_blocks += __builtin_amdgcn_readlane(incl, kWave - 1);
  }
  if (wid == 0 && lane == 0) p.cum_blocks[0] = 0;
  const int64_t n_tiles = total_blocks * p.pairs_per_seq;
  const int64_t chunk = chunk_tiles(p, n_tiles);
  const int64_t t0 = wid * chunk;
  if (t0 >= n_tiles) return false;
  left = (t0 + chunk < n_tiles ? t0 + chunk : n_tiles) - t0;

  int64_t before = 0;  // blocks of the sequences scanned so far
  c.seq = p.n_seqs;
  c.nb = 1;
  int cum = 0;
  for (int base = 0; base < p.n_seqs; base += kWave) {
    const int s = base + lane;
    const int mine = s < p.n_seqs ? seq_blocks(p, s, BS) : 0;
    const int incl = wave_inclusive_scan(mine, lane);
    // first sequence whose tiles end after t0
    const uint64_t hit = __ballot((before + incl) * p.pairs_per_seq > t0);
    if (hit != 0) {
      const int ln = __builtin_ctzll(hit);
      c.seq = base + ln;
      c.nb = __builtin_amdgcn_readlane(mine, ln);
      cum = (int)(before + __builtin_amdgcn_readlane(incl, ln)) - c.nb;
      break;
    }
    before += __builtin_amdgcn_readlane(incl, kWave - 1);
  }
  const int64_t r = t0 - (int64_t)cum * p.pairs_per_seq;
  c.pair = (int)(r / c.nb);
  c.blk = (int)(r - (int64_t)c.pair * c.nb);
  return true;
}

// Window = the next n_win (<= 64*SW) tiles of the share.  Each lane looks up
// the pool block of SW of them and keeps the tile's byte offset (the same for
// the K and the V pool); `walk` advances past the window.
template <int BS, int SW, int ES>
__device__ __forceinline__ void gather_window(const DecodeKP &p, int lane, int n_win, TileCursor &walk,
                                              uint32_t *off_lo, uint32_t *off_hi) {
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
    const int64_t row = (int64_t)walk.seq * p.bt_stride;
#pragma unroll
    for (int r = 0; r < SW; ++r) {
      const int lp = r * kWave + lane;
      const bool in = lp >= pos && lp < pos + cnt;
      int tile_in_seq = walk.blk + lp - pos;
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
    if (walk.blk == walk.nb) next_pair<BS>(p, walk);
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

// Launches the query-group decode main kernel (paged_decode_mfma.hip) when it is
// built for this shape; returns false otherwise.  Sets kp.n_waves.
bool launch_decode_mfma_main(DecodeKP &kp, int dtype, int hd, int gt, hipStream_t stream);

}  // namespace decode
}  // namespace ic
