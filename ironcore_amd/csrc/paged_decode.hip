// Paged decode: one query token per sequence against the block KV cache.
//
// What it computes is the reference's dense attention with sq = 1
// (ironcore/layers/attention.py:68-142) on the rows the block table names:
// scores = q.k * scale, softmax over the context, out = probs @ v, with query
// head h reading KV head h / G (attention.py:95-102).
//
// This file holds the host-side launch, the split-K reduce pass and the
// vector-ALU main kernel, which is the one fp32 pools run on (scores, softmax
// and the PV sum stay in fp32).  bf16 and fp16 pools take the matrix-core main
// kernel of paged_decode_mfma.hip; both share everything described here
// except the arithmetic of a tile.
//
// HBM-bound streaming kernel (one pass over every visible K and V byte).
//
//  * Unit of work: a TILE = 16 consecutive tokens of one (sequence, KV head)
//    "pair" (one pool block at block size 16, a slice of a longer block
//    otherwise), for ALL G query heads that share the KV head, so each K/V
//    byte is fetched once per KV head, not once per query head.  (G > 8 is
//    cut into sub-groups of <= 8 heads, each its own pair.)
//  * Split-K by equal shares: the tiles of the whole batch form one sequence
//    (pair-major, block-minor); every resident WAVE prefix-sums the
//    per-sequence block counts and takes one contiguous chunk of
//    ceil(N / waves) tiles.  A chunk may start and end inside a pair and may
//    span several pairs; each (wave, pair) segment yields one partial.  All
//    waves carry the same load whatever the spread of context lengths, the
//    grid is exactly the number of waves the GPU holds at once, and waves
//    never synchronise with each other.  Shares are dealt XCD-major, so
//    neighbouring shares (which may alias the same prefix blocks) share an L2.
//  * At the start of its chunk a wave gathers the byte offsets of its next
//    256 tiles from the block table, one per lane and slot; the loop reads
//    them back as wave-uniform scalars (v_readlane), so the table is off the
//    load path and tile addresses are SALU work.
//  * One tile is block_size*hd contiguous elements per K and per V; each lane
//    fetches 16 bytes per load, so one load instruction covers 1 KiB of
//    consecutive bytes (64/LPR token rows, LPR = lanes per row).  Two
//    register tiles in ping-pong: the next tile's loads are in flight while
//    the current one is consumed, across pair boundaries too; the next
//    pair's query is prefetched a segment ahead.
//  * q.k: fused multiply-adds (v_dot2 for 16-bit types), then a DPP butterfly
//    over the LPR lanes that share a row.  Online softmax per lane group; p*v
//    accumulates into EPL fp32 registers per query head with no cross-lane
//    traffic.
//  * Segment end: the lane groups of the wave are merged (log-sum-exp) through
//    a private LDS slab.  A segment that covers its whole pair writes the
//    output row; otherwise (m, l, acc) go to the workspace and the reduce
//    kernel combines the few partials of that pair.
//
// Algorithmic bytes per launch: sum_i ctx_i * 2 * gn * hd * elem (K and V,
// once per KV head) + q, out, block-table entries and context lengths.
#include "decode_common.h"
#include "../../include/ironcore_paged.h"

namespace ic {

using namespace decode;

namespace {

template <class E, int HD, int GT, int BS, int NW>
__global__ __launch_bounds__(NW *kWave) void paged_decode_kernel(const DecodeKP p) {
  using T = typename E::type;
  constexpr int EPL = E::EPL;
  constexpr int ES = sizeof(T);
  constexpr int LPR = HD / EPL;     // lanes sharing one token row
  constexpr int RPL = kWave / LPR;  // token rows per load instruction
  constexpr int NLD = BS / RPL;     // load instructions per tile
  constexpr int SW = 4;             // tile offsets held per lane: a window is 64*SW tiles
  static_assert(HD % EPL == 0 && kWave % LPR == 0 && BS % RPL == 0, "tile shape");

  __shared__ __attribute__((aligned(16))) float s_acc[NW][RPL][GT][HD];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int col = lane % LPR;
  const int rowg = lane / LPR;

  // ---- this wave's share of the batch-wide tile sequence ----------------------
  const int64_t wid = (int64_t)xcd_major_workgroup() * NW + wave;
  int64_t left;  // tiles not yet consumed
  TileCursor c;
  if (!locate_chunk<BS>(p, lane, 0, wid, left, c)) return;
  TileCursor walk = c;  // gathers tile addresses ahead of the arithmetic
  TileCursor peek = c;  // the segment after the current one (its q is prefetched)
  next_pair(p, GlobalRows<BS>{p, 0}, peek);
  int seg_blk0 = c.blk;

  uint32_t lane_off[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i)
    lane_off[i] = (uint32_t)(((i * RPL + rowg) * p.stride_token + col * EPL) * ES);

  auto load_q = [&](const TileCursor &tc, Vec16 *qq) {
    const int kvh = tc.pair / p.nsub;
    const int sub = tc.pair - kvh * p.nsub;
    const int head0 = kvh * p.group + sub * GT;
    const int heads = (p.group - sub * GT < GT) ? p.group - sub * GT : GT;
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      qq[g] = Vec16{{0u, 0u, 0u, 0u}};
      if (g < heads && tc.seq < p.n_seqs)
        qq[g] = load16(p.q + (tc.seq * p.q_stride_seq + (int64_t)(head0 + g) * HD + col * EPL) * ES);
    }
  };
  Vec16 qreg[GT], qnext[GT];
  load_q(c, qreg);
  load_q(peek, qnext);

  float m[GT], l[GT], acc[GT][EPL];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = kNegInf;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
  }

  // End of a segment: merge the RPL row groups of the wave (log-sum-exp)
  // through the wave's LDS slab, write the output row or a partial, then move
  // to the next pair.  The next tile's loads are already in flight.
  auto finish_segment = [&]() {
    const int kvh = c.pair / p.nsub;
    const int sub = c.pair - kvh * p.nsub;
    const int head0 = kvh * p.group + sub * GT;
    const int heads = (p.group - sub * GT < GT) ? p.group - sub * GT : GT;
    float lsum[GT], mall[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      float mx = m[g];
      if (RPL >= 2) mx = fmaxf(mx, __shfl_xor(mx, LPR, kWave));
      if (RPL >= 4) mx = fmaxf(mx, __shfl_xor(mx, 2 * LPR, kWave));
      if (RPL >= 8) mx = fmaxf(mx, __shfl_xor(mx, 4 * LPR, kWave));
      const float w = (m[g] == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m[g] - mx);
      float ls = l[g] * w;
      if (RPL >= 2) ls += __shfl_xor(ls, LPR, kWave);
      if (RPL >= 4) ls += __shfl_xor(ls, 2 * LPR, kWave);
      if (RPL >= 8) ls += __shfl_xor(ls, 4 * LPR, kWave);
      lsum[g] = ls;
      mall[g] = mx;
#pragma unroll
      for (int e = 0; e < EPL; e += 4) {
        float4 v4 = make_float4(acc[g][e] * w, acc[g][e + 1] * w, acc[g][e + 2] * w, acc[g][e + 3] * w);
        *reinterpret_cast<float4 *>(&s_acc[wave][rowg][g][col * EPL + e]) = v4;
      }
      m[g] = kNegInf;
      l[g] = 0.f;
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
    }
    // Only this wave reads what it wrote: a wave-level fence is enough.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool whole_pair = (seg_blk0 == 0 && c.blk == c.nb);
    const int64_t partial = wid + (int64_t)c.seq * p.pairs_per_seq + c.pair;
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (g >= heads) break;
      const int h = head0 + g;
#pragma unroll
      for (int d = lane; d < HD; d += kWave) {
        float a = 0.f;
#pragma unroll
        for (int r = 0; r < RPL; ++r) a += s_acc[wave][r][g][d];
        if (whole_pair)
          reinterpret_cast<T *>(p.out)[c.seq * p.out_stride_seq + (int64_t)h * HD + d] =
              E::narrow(a / lsum[g]);
        else
          p.part_acc[(partial * GT + g) * HD + d] = a;
      }
      if (!whole_pair && lane == 0) {
        p.part_ml[(partial * GT + g) * 2] = mall[g];
        p.part_ml[(partial * GT + g) * 2 + 1] = lsum[g];
      }
    }
    // The slab is reused by the next segment.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (left > 0) {
      c = peek;
      seg_blk0 = 0;
#pragma unroll
      for (int g = 0; g < GT; ++g) qreg[g] = qnext[g];
      next_pair(p, GlobalRows<BS>{p, 0}, peek);
      load_q(peek, qnext);
    }
  };

  // One tile of arithmetic on the registers (kk, vv), for the tile at cursor c.
  auto consume = [&](Vec16 *kk, Vec16 *vv) {
    float s[GT][NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        float d = E::dot(kk[i], qreg[g], 0.f);
        s[g][i] = group_sum<LPR>(d) * p.scale_log2e;
      }
    }
    if (c.blk == c.nb - 1) {  // the sequence's last block may be partly filled
      int ctx = p.context_lens[c.seq];
      ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
      const int tok0 = c.blk * BS;
      if (tok0 + BS > ctx) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
          if (tok0 + i * RPL + rowg >= ctx) {
#pragma unroll
            for (int g = 0; g < GT; ++g) s[g][i] = kNegInf;
            vv[i] = Vec16{{0u, 0u, 0u, 0u}};
          }
        }
      }
    }
    if (p.key_mask != nullptr) {  // keys the caller's mask hides (context-length cuts stay -inf)
      int ctx = p.context_lens[c.seq];
      ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
      const int kvh = c.pair / p.nsub;
      const int head0 = kvh * p.group + (c.pair - kvh * p.nsub) * GT;
      const uint8_t *mrow = p.key_mask + c.seq * p.key_mask_stride_seq + c.blk * BS + rowg;
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        if (c.blk * BS + i * RPL + rowg < ctx) {
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            const int h = head0 + g < p.hn ? head0 + g : p.hn - 1;
            if (mrow[h * p.key_mask_stride_head + i * RPL] == 0) s[g][i] = kHiddenLog2;
          }
        }
      }
    }
    float vf[NLD][EPL];
#pragma unroll
    for (int i = 0; i < NLD; ++i) E::widen(vv[i], vf[i]);
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      float mx = m[g];
#pragma unroll
      for (int i = 0; i < NLD; ++i) mx = fmaxf(mx, s[g][i]);
      const float ms = (mx == kNegInf) ? 0.f : mx;
      const float alpha = __builtin_amdgcn_exp2f(m[g] - ms);
      float pr[NLD];
      float ps = 0.f;
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        pr[i] = __builtin_amdgcn_exp2f(s[g][i] - ms);
        ps += pr[i];
      }
      l[g] = l[g] * alpha + ps;
      m[g] = mx;
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        float a = acc[g][e] * alpha;
#pragma unroll
        for (int i = 0; i < NLD; ++i) a = __builtin_fmaf(pr[i], vf[i][e], a);
        acc[g][e] = a;
      }
    }
    ++c.blk;
    --left;
    if (c.blk == c.nb || left == 0) finish_segment();
  };

  while (left > 0) {
    // ---- window: byte offsets of the next n_win tiles, one per lane and slot ---
    const int n_win = left < kWave * SW ? (int)left : kWave * SW;
    uint32_t off_lo[SW], off_hi[SW];
    gather_window<BS, SW, ES>(p, GlobalRows<BS>{p, 0}, lane, n_win, walk, off_lo, off_hi);

    auto issue = [&](int i, Vec16 *kk, Vec16 *vv) {
      const int64_t tile = window_tile_offset(off_lo, off_hi, i);
      const char *kb = p.k_pool + tile;
      const char *vb = p.v_pool + tile;
#pragma unroll
      for (int q4 = 0; q4 < NLD; ++q4) kk[q4] = load16(kb + lane_off[q4]);
#pragma unroll
      for (int q4 = 0; q4 < NLD; ++q4) vv[q4] = load16(vb + lane_off[q4]);
      // Keep the loads ahead of the arithmetic that follows in program order:
      // the scheduler would otherwise sink them below the current tile's work
      // and shorten the prefetch distance.
      __builtin_amdgcn_sched_barrier(0);
    };

    // Two register tiles in ping-pong.  The steady-state loop issues the next
    // tile's loads unconditionally, so the wait before a tile is consumed
    // covers that tile only and the prefetch stays in flight behind it,
    // across pair boundaries too.
    Vec16 ka[NLD], va[NLD], kb[NLD], vb[NLD];
    int i = 0;
    issue(0, ka, va);
    for (; i + 2 < n_win; i += 2) {
      issue(i + 1, kb, vb);
      consume(ka, va);
      issue(i + 2, ka, va);
      consume(kb, vb);
    }
    if (i + 2 == n_win) {
      issue(i + 1, kb, vb);
      consume(ka, va);
      consume(kb, vb);
    } else {
      consume(ka, va);
    }
  }
}

constexpr int kReduceThreads = 256;

// Combine the split-K partials of one pair (a KV head's query heads of one
// sequence).  grid = (pairs per sequence / pairs per workgroup, n_seqs).  A pair's tiles in a row
// are a contiguous run of a phase's tile sequence, so the shares that touched
// it are first_tile / chunk .. last_tile / chunk and their partial ids follow.
// With shared-prefix cohorts a sequence has two sources: its own row and its
// cohort's row of the shared phase, where it owns `group` of the matrix
// columns of one wave of each unit.
// Traffic is (hd+2)*4 bytes per partial, three orders of magnitude below the
// K/V stream; what costs time here is the chain of dependent memory round
// trips, so the prefix sums are fetched together and every thread fetches up
// to four partials of its four output dims in one batch before it merges them
// (a typical pair has two to four partials: two round trips in all).
template <class E, int HD>
__global__ __launch_bounds__(kReduceThreads) void paged_decode_reduce_kernel(const DecodeKP p) {
  using T = typename E::type;
  constexpr int QPH = HD / 4;  // 4-dim groups per head row
  constexpr int UB = 4;        // partials fetched per batch
  const int COLS = p.gt;
  // A pair keeps COLS * QPH threads busy; a workgroup takes as many pairs of
  // its sequence as fit (8 for MHA at hd 128), each on its own slice of threads.
  const int width = COLS * QPH < kReduceThreads ? COLS * QPH : kReduceThreads;
  const int per_wg = kReduceThreads / width;
  const int tid = threadIdx.x % width;
  const int pair_in_seq = blockIdx.x * per_wg + threadIdx.x / width;
  const int seq = blockIdx.y;
  if (pair_in_seq >= p.pairs_per_seq || threadIdx.x >= per_wg * width) return;
  const int kvh = pair_in_seq / p.nsub;
  const bool cohorts = p.cohort_size > 1;
  int heads, head0, cohort = 0, col_sh = 0, wave_sh = 0;
  if (!cohorts) {
    const int sub = pair_in_seq - kvh * p.nsub;
    head0 = kvh * p.group + sub * COLS;
    heads = (p.group - sub * COLS < COLS) ? p.group - sub * COLS : COLS;
  } else {
    cohort = seq / p.cohort_size;
    const int u = seq - cohort * p.cohort_size;
    wave_sh = u / p.spw;                        // the wave of a unit that carries this member
    col_sh = (u - wave_sh * p.spw) * p.group;   // its first column there
    head0 = kvh * p.group;
    heads = p.group;
  }
  const int cum_own = p.cum_blocks[seq];
  const int nb_own = p.cum_blocks[seq + 1] - cum_own;
  const int cum_all = p.cum_blocks[p.n_seqs];
  int cum_sh = 0, nb_sh = 0, cum_sh_all = 0;
  if (cohorts) {
    cum_sh = p.cum_shared[cohort];
    nb_sh = p.cum_shared[cohort + 1] - cum_sh;
    cum_sh_all = p.cum_shared[p.n_cohorts];
  }
  T *orow = reinterpret_cast<T *>(p.out) + seq * p.out_stride_seq + (int64_t)head0 * HD;
  if (nb_own + nb_sh == 0) {  // no visible token: zero rows
    for (int o = tid; o < heads * HD; o += width) orow[o] = E::narrow(0.f);
    return;
  }
  // source 0: the cohort's row of the shared phase, source 1: the sequence's
  // own row; an empty source gets an empty share range.  A share w of a source
  // left its partial in slot (w + slot0) * mul + add, column col0 + g.
  int64_t w_lo[2], w_hi[2], slot0[2], mul[2], add[2];
  int col0[2];
  {
    const int64_t chunk = chunk_tiles(p, (int64_t)cum_sh_all * p.pairs_per_seq, phase_units(p, 1));
    const int64_t first = (int64_t)cum_sh * p.pairs_per_seq + (int64_t)pair_in_seq * nb_sh;
    w_lo[0] = first / chunk;
    w_hi[0] = nb_sh > 0 ? (first + nb_sh - 1) / chunk : w_lo[0] - 1;
    slot0[0] = (int64_t)cohort * p.pairs_per_seq + pair_in_seq;
    mul[0] = (int64_t)1 << p.unit_shift;
    add[0] = p.shared_slot0 + wave_sh;
    col0[0] = col_sh;
  }
  {
    const int64_t chunk = chunk_tiles(p, (int64_t)cum_all * p.pairs_per_seq, phase_units(p, 0));
    const int64_t first = (int64_t)cum_own * p.pairs_per_seq + (int64_t)pair_in_seq * nb_own;
    w_lo[1] = first / chunk;
    w_hi[1] = nb_own > 0 ? (first + nb_own - 1) / chunk : w_lo[1] - 1;
    slot0[1] = (int64_t)seq * p.pairs_per_seq + pair_in_seq;
    mul[1] = 1;
    add[1] = 0;
    col0[1] = 0;
  }
  // one wave covered all the sequence has for this pair and wrote the rows
  if (nb_sh == 0 && w_lo[1] == w_hi[1]) return;
  for (int o = tid; o < heads * QPH; o += width) {
    const int g = o / QPH;
    const int d = (o - g * QPH) * 4;
    float m_run = kNegInf, l_run = 0.f;
    float4 a_run = make_float4(0.f, 0.f, 0.f, 0.f);
    // the partials of both sources as one list, fetched UB at a time: all loads of a batch are
    // independent and in flight together, whichever source they come from
    const int64_t n0 = w_hi[0] - w_lo[0] + 1, n_all = n0 + (w_hi[1] - w_lo[1] + 1);
    for (int64_t ib = 0; ib < n_all; ib += UB) {
      float2 ml[UB];
      float4 av[UB];
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        const int64_t i = ib + u < n_all ? ib + u : n_all - 1;
        const int src = i < n0 ? 0 : 1;
        const int64_t w = src == 0 ? w_lo[0] + i : w_lo[1] + (i - n0);
        const int64_t slot = ((w + slot0[src]) * mul[src] + add[src]) * COLS + col0[src] + g;
        ml[u] = *reinterpret_cast<const float2 *>(p.part_ml + slot * 2);
        av[u] = *reinterpret_cast<const float4 *>(p.part_acc + slot * HD + d);
      }
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        if (ib + u >= n_all || ml[u].x == kNegInf) continue;
        const float m_new = fmaxf(m_run, ml[u].x);
        const float keep = (m_run == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
        const float wt = __builtin_amdgcn_exp2f(ml[u].x - m_new);
        l_run = __builtin_fmaf(ml[u].y, wt, l_run * keep);
        a_run.x = __builtin_fmaf(av[u].x, wt, a_run.x * keep);
        a_run.y = __builtin_fmaf(av[u].y, wt, a_run.y * keep);
        a_run.z = __builtin_fmaf(av[u].z, wt, a_run.z * keep);
        a_run.w = __builtin_fmaf(av[u].w, wt, a_run.w * keep);
        m_run = m_new;
      }
    }
    const float inv = 1.f / l_run;
    T *dst = orow + g * HD + d;
    dst[0] = E::narrow(a_run.x * inv);
    dst[1] = E::narrow(a_run.y * inv);
    dst[2] = E::narrow(a_run.z * inv);
    dst[3] = E::narrow(a_run.w * inv);
  }
}

// Waves of the main kernel that one GPU holds at once, per kernel variant.
template <class E, int HD, int GT, int BS, int NW>
int resident_workgroups() {
  static const int per_cu = [] {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, paged_decode_kernel<E, HD, GT, BS, NW>,
                                                     NW * kWave, 0) != hipSuccess || n < 1)
      n = 1;
    return n;
  }();
  return per_cu * device_cu_count();
}

template <class E, int HD>
int launch_reduce(const DecodeKP &kp, hipStream_t stream) {
  const int width = kp.gt * (HD / 4) < kReduceThreads ? kp.gt * (HD / 4) : kReduceThreads;
  const int per_wg = kReduceThreads / width;  // pairs per workgroup, as the kernel derives it
  hipLaunchKernelGGL((paged_decode_reduce_kernel<E, HD>), dim3((kp.pairs_per_seq + per_wg - 1) / per_wg, kp.n_seqs),
                     dim3(kReduceThreads), 0, stream, kp);
  return hipGetLastError() == hipSuccess ? IC_OK : IC_ERR_LAUNCH;
}

// fp32 pools: the vector-ALU main kernel, one instantiation per group size.
template <class E, int HD, int GT>
void launch_valu_main(DecodeKP &kp, hipStream_t stream) {
  constexpr int BS = 16;
  constexpr int NW = kDecodeWavesPerWorkgroup;
  int wgs = resident_workgroups<E, HD, GT, BS, NW>();
  if (wgs * NW > kp.max_waves) wgs = kp.max_waves / NW;
  kp.n_waves = wgs * NW;
  hipLaunchKernelGGL((paged_decode_kernel<E, HD, GT, BS, NW>), dim3(wgs), dim3(NW * kWave), 0, stream, kp);
}

template <class E, int HD>
int launch_group(DecodeKP &kp, int dtype, hipStream_t stream) {
  if constexpr (sizeof(typename E::type) == 2) {
    // 16-bit element types: the matrix-core kernel, whatever the group size.
    if (!launch_decode_mfma_main(kp, dtype, HD, stream)) return IC_ERR_UNSUPPORTED;
  } else {
    if (kp.cohort_size != 1) return IC_ERR_UNSUPPORTED;
    switch (kp.gt) {
      case 1: launch_valu_main<E, HD, 1>(kp, stream); break;
      case 2: launch_valu_main<E, HD, 2>(kp, stream); break;
      case 3: launch_valu_main<E, HD, 3>(kp, stream); break;
      case 4: launch_valu_main<E, HD, 4>(kp, stream); break;
      case 5: launch_valu_main<E, HD, 5>(kp, stream); break;
      case 6: launch_valu_main<E, HD, 6>(kp, stream); break;
      case 7: launch_valu_main<E, HD, 7>(kp, stream); break;
      default: launch_valu_main<E, HD, 8>(kp, stream); break;
    }
  }
  return launch_reduce<E, HD>(kp, stream);
}

template <class E>
int launch_hd(DecodeKP &kp, int hd, int dtype, hipStream_t stream) {
  switch (hd) {
    case 32: return launch_group<E, 32>(kp, dtype, stream);
    case 64: return launch_group<E, 64>(kp, dtype, stream);
    case 128: return launch_group<E, 128>(kp, dtype, stream);
    default: return IC_ERR_UNSUPPORTED;
  }
}

}  // namespace

int launch_paged_decode(const DecodeArgs &a, hipStream_t stream) {
  // The kernel loads whole 16-token tiles, so a pool block must hold a whole
  // number of them (a tile never straddles the end of a block).
  if (a.pool.block_size % 16 != 0) return IC_ERR_UNSUPPORTED;
  DecodeKP kp;
  kp.q = (const char *)a.q;
  kp.k_pool = (const char *)a.k_pool;
  kp.v_pool = (const char *)a.v_pool;
  kp.block_tables = a.block_tables;
  kp.context_lens = a.context_lens;
  kp.out = (char *)a.out;
  kp.cum_blocks = a.cum_blocks;
  kp.part_ml = a.part_ml;
  kp.part_acc = a.part_acc;
  kp.q_stride_seq = a.q_stride_seq;
  kp.out_stride_seq = a.out_stride_seq;
  kp.stride_block = a.pool.stride_block;
  kp.stride_head = a.pool.stride_head;
  kp.stride_token = a.pool.stride_token;
  kp.bt_stride = a.block_table_stride;
  kp.num_blocks = a.pool.num_blocks;
  kp.n_seqs = a.n_seqs;
  kp.hn = a.hn;
  kp.group = a.hn / a.gn;
  const DecodeLayout lay = decode_layout(a.n_seqs, a.hn, a.gn, a.cohort_size);
  if (!lay.ok) return IC_ERR_UNSUPPORTED;
  kp.nsub = lay.nsub;
  kp.gt = lay.cols;
  kp.pairs_per_seq = a.gn * lay.nsub;
  kp.cohort_size = a.cohort_size > 1 ? a.cohort_size : 1;
  kp.cohort_shared = a.cohort_size > 1 ? a.cohort_shared_blocks : nullptr;
  kp.n_cohorts = lay.n_cohorts;
  kp.spw = lay.spw;
  kp.unit_shift = lay.unit_shift;
  kp.cum_shared = a.cum_blocks + a.n_seqs + 1;
  kp.shared_slot0 = a.shared_slot0;
  kp.max_ctx = a.max_context_len;
  kp.n_waves = 0;
  kp.max_waves = a.max_waves > 0 && a.max_waves < kMaxDecodeWaves ? a.max_waves : kMaxDecodeWaves;
  kp.min_chunk = (a.min_chunk_tokens + 15) / 16;
  kp.tiles_per_block = a.pool.block_size / 16;
  kp.scale_log2e = a.scale * 1.4426950408889634f;
  kp.key_mask = a.key_mask;
  kp.key_mask_stride_seq = a.key_mask_stride_seq;
  kp.key_mask_stride_head = a.key_mask_stride_head;
  if (a.key_mask != nullptr && a.dtype != IC_DTYPE_F32) return IC_ERR_UNSUPPORTED;
  switch (a.dtype) {
    case IC_DTYPE_BF16: return launch_hd<Bf16>(kp, a.hd, a.dtype, stream);
    case IC_DTYPE_F16: return launch_hd<F16>(kp, a.hd, a.dtype, stream);
    case IC_DTYPE_F32: return launch_hd<F32>(kp, a.hd, a.dtype, stream);
    default: return IC_ERR_UNSUPPORTED;
  }
}

}  // namespace ic
