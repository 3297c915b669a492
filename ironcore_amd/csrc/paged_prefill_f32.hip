// Chunked prefill against the block KV cache for fp32 pools.
//
// Same contract as the 16-bit kernel of paged_prefill.hip (the reference's
// dense attention, ironcore/layers/attention.py:68-142, with sq = C, sk = L
// and the causal mask of ironcore/language_model.py:109-114 shifted by the
// cached prefix, no mask, or a caller's byte mask), with every product, sum
// and probability in fp32: the dtype the reference's own contract tests feed
// the layer (tests/test_attention.py:143-161).
//
// Flash-attention shape on the fp32 matrix instruction (v_mfma_f32_32x32x2_f32):
//
//  * One workgroup = 128 query rows of one query head: 4 waves, each owning 32
//    rows for the whole K/V sweep.  The wave's query rows stay in registers as
//    MFMA B operands.
//  * K/V are walked in tiles of 32 tokens.  All 256 threads fetch a tile from
//    the pool through the block table (16 bytes per lane and load, rows past
//    the context clamped to the last one) a whole tile ahead, hold it in
//    registers while the current tile is computed, then leave it in the other
//    of two LDS buffers: a K/V byte crosses the memory system once per 128
//    query rows, and there is one workgroup barrier per tile.
//  * S^T = K Q^T: a lane supplies K[token lane % 32][d] and Q[query lane % 32][d]
//    for one d per MFMA; the k index of MFMA 4j + e is d = 8j + 4(lane / 32) + e,
//    so that a lane's four operands of a group are one 16-byte LDS read.  K rows
//    are padded by 4 floats, which spreads the 16 rows of an access over all
//    banks.  A lane then holds one query column of the scores: row maximum and
//    row sum are in-lane reductions plus one exchange between the lane halves.
//  * O^T += V^T P^T: the probabilities are already B operands (MFMA i of a
//    lane half takes the token that half holds in register i), the matching
//    V^T operand is one float per lane from the row-major V tile (rows padded
//    by 8 floats: the two halves read rows 4 apart, on disjoint banks).
//  * Tiles wholly above the causal diagonal are skipped per wave.
//
// FLOPs per launch: 4*hn*hd per visible (query, key) pair, as for the 16-bit
// kernel; bound by the fp32 matrix rate (157 TFLOP/s nominal).
#include "prefill_common.h"
#include "../../include/ironcore_paged.h"

namespace ic {
namespace prefill {

namespace {

constexpr int kF32Waves = 4;
constexpr int kF32Threads = kF32Waves * kWave;
constexpr int kF32BM = kF32Waves * 32;  // query rows per workgroup
constexpr int kF32BN = 32;              // tokens per K/V tile

template <int HD, bool SINGLE, bool MASK>
__global__ __launch_bounds__(kF32Threads) void paged_prefill_f32_kernel(const PrefillKP p) {
  constexpr int NJ = HD / 8;            // 16-byte operand groups of the QK contraction
  constexpr int OB = HD / 32;           // 32-wide blocks of the output head dim
  constexpr int F4R = HD / 4;           // 16-byte pieces per token row
  constexpr int RP = kF32Threads / F4R; // token rows one pass of the workgroup covers
  constexpr int NP = kF32BN / RP;       // passes (pieces per thread and pool) per tile
  constexpr int KP = HD + 4;            // LDS row pitch of K, floats
  constexpr int VP = HD + 8;            // ... of V
  static_assert(HD % 32 == 0 && kF32Threads % F4R == 0 && kF32BN % RP == 0 && NP >= 1, "tile staging shape");

  __shared__ __attribute__((aligned(16))) float s_k[2][kF32BN * KP];
  __shared__ __attribute__((aligned(16))) float s_v[2][kF32BN * VP];

  const int seq = blockIdx.y;
  const int h = blockIdx.x / p.n_qtiles;
  const int q0 = (p.n_qtiles - 1 - blockIdx.x % p.n_qtiles) * kF32BM;  // last query tiles (the longest) first
  const int kvh = h / p.group;
  const int q_lo = p.cu_seqlens_q[seq];
  int L = p.context_lens[seq];
  int C = p.cu_seqlens_q[seq + 1] - q_lo;
  const bool causal = !MASK && p.causal;
  if (L < 0) L = 0;
  if (causal && C > L) C = L;  // under the causal rule a chunk cannot be longer than its context
  if (q0 >= C) return;
  const int tid = threadIdx.x;
  if (L == 0) {  // query rows without any key (not under the causal rule): zero rows
    const int rows = C - q0 < kF32BM ? C - q0 : kF32BM;
    for (int idx = tid; idx < rows * F4R; idx += kF32Threads)
      store16(p.out + ((q_lo + q0 + idx / F4R) * p.out_stride_token + (int64_t)h * HD + (idx % F4R) * 4) * 4,
              Vec16{{0u, 0u, 0u, 0u}});
    return;
  }
  const int P = L - C;  // cached prefix (causal rule only)
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int n = lane & 31;   // query column of this lane within the wave's 32-row block
  const int hh = lane >> 5;  // which operand of each k pair this lane feeds

  // ---- query rows: registers for the whole sweep, as MFMA B operands ------------
  const int my_q = q0 + wave * 32 + n;
  const int qrow = my_q < C ? my_q : C - 1;
  const int limit = causal ? P + qrow : L - 1;  // last key this query row may see
  float4 qf[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
    qf[j] = *reinterpret_cast<const float4 *>(
        p.q + ((q_lo + qrow) * p.q_stride_token + (int64_t)h * HD + 8 * j + 4 * hh) * 4);

  f32x16_t o[OB];
  float m = kNegInf, l = 0.f;
#pragma unroll
  for (int ob = 0; ob < OB; ++ob)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[ob][i] = 0.f;

  int kv_end = causal ? P + q0 + kF32BM : L;  // keys any row of this workgroup can see
  kv_end = kv_end < L ? kv_end : L;
  const int n_tiles = (kv_end + kF32BN - 1) / kF32BN;
  int my_end = causal ? P + q0 + wave * 32 + 32 : L;
  my_end = my_end < kv_end ? my_end : kv_end;
  const int my_tiles = (my_end > 0 && q0 + wave * 32 < C) ? (my_end + kF32BN - 1) / kF32BN : 0;

  // ---- tile staging: memory -> registers (a tile ahead) -> LDS -------------------------
  const int r0 = tid / F4R;  // first token row of the tile this thread fetches
  const int c4 = tid % F4R;  // its 16-byte piece of the row
  const int32_t *table_row = p.block_tables + (int64_t)seq * p.bt_stride;
  const int64_t head_off = (int64_t)kvh * p.stride_head + c4 * 4;
  auto fetch = [&](int tile, Vec16 *kr, Vec16 *vr) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      int tok = tile * kF32BN + r0 + i * RP;
      tok = tok < L ? tok : L - 1;  // rows past the context: a valid row, never visible
      int blk = 0, within = tok;
      if (!SINGLE) {
        blk = p.block_shift >= 0 ? tok >> p.block_shift : tok / p.block_size;
        within = tok - blk * p.block_size;
      }
      int64_t phys = table_row[blk];
      // A corrupt table entry must not become an out-of-pool address.
      phys = phys < 0 ? 0 : phys;
      phys = phys >= p.num_blocks ? p.num_blocks - 1 : phys;
      const int64_t off = (phys * p.stride_block + head_off + (int64_t)within * p.stride_token) * 4;
      kr[i] = load16(p.k_pool + off);
      vr[i] = load16(p.v_pool + off);
    }
  };
  auto stash = [&](int buf, const Vec16 *kr, const Vec16 *vr) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      store16(&s_k[buf][(r0 + i * RP) * KP + c4 * 4], kr[i]);
      store16(&s_v[buf][(r0 + i * RP) * VP + c4 * 4], vr[i]);
    }
  };

  f32x16_t s;  // S^T of the tile: (token, query n); after the softmax its probabilities

  // ---- S^T = K Q^T ----------------------------------------------------------------
  auto scores = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    const float *kb = &s_k[buf][n * KP + 4 * hh];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const float4 a = *reinterpret_cast<const float4 *>(kb + 8 * j);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, qf[j].x, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, qf[j].y, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, qf[j].z, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, qf[j].w, s, 0, 0, 0);
    }
  };
  // ---- softmax of the tile's scores: s -> probabilities, m, l (and o when the reference moves) ----
  auto softmax = [&](int tile) {
    // s[i] is (token tile*32 + 4*hh + 8*(i/4) + i%4, query n)
    const int tok_base = tile * kF32BN + 4 * hh;
    const bool need_mask = causal ? (tile * kF32BN + kF32BN - 1 > P + q0 + wave * 32) : (tile * kF32BN + kF32BN > L);
    if (need_mask) {  // tiles that touch the causal diagonal (or the context end)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int tok = tok_base + 8 * (i / 4) + (i & 3);
        s[i] = tok > limit ? kNegInf : s[i];
      }
    }
    if constexpr (MASK) {  // keys the caller's mask hides from this lane's query row
      const uint8_t *mrow = p.mask + (int64_t)seq * p.mask_stride_seq + (int64_t)h * p.mask_stride_head +
                            (int64_t)qrow * p.mask_stride_row;
      // unconditional loads from an index clamped into the part of the row that exists and counts
      const int last = (limit < p.mask_keys - 1 ? limit : p.mask_keys - 1);
      uint8_t seen[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int tok = tok_base + 8 * (i / 4) + (i & 3);
        seen[i] = mrow[tok < last ? tok : last];
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int tok = tok_base + 8 * (i / 4) + (i & 3);
        const bool hidden = (tok <= limit) & ((tok >= p.mask_keys) | (seen[i] == 0));
        s[i] = hidden ? kHiddenScore : s[i];
      }
    }
    float mx = kNegInf;
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[i]);
    float mx_a, mx_b;
    both_halves(mx, mx_a, mx_b);
    mx = fmaxf(mx_a, mx_b) * p.scale_log2e;
    // Lazy reference maximum, as in the 16-bit kernel: it moves (and the accumulators are
    // rescaled) only when some row's maximum rises more than 2^kLazySlack above it.
    if (__any(mx > m + kLazySlack)) {
      const float m_new = fmaxf(m, mx);
      const float alpha = (m == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
      m = m_new;
      l *= alpha;
#pragma unroll
      for (int ob = 0; ob < OB; ++ob)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[ob][i] *= alpha;
    }
    const float neg_ms = (m == kNegInf) ? 0.f : -m;
    float ps = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], p.scale_log2e, neg_ms));
      ps += s[i];
    }
    l += ps;
  };
  // ---- O^T += V^T P^T ---------------------------------------------------------------
  auto weighted_values = [&](int buf) {
    const float *vb = &s_v[buf][4 * hh * VP + n];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float *row = vb + ((i & 3) + 8 * (i >> 2)) * VP;  // token (i%4) + 8(i/4) + 4hh of the tile
#pragma unroll
      for (int ob = 0; ob < OB; ++ob) o[ob] = __builtin_amdgcn_mfma_f32_32x32x2f32(row[ob * 32], s[i], o[ob], 0, 0, 0);
    }
  };

  Vec16 kr[NP], vr[NP];
  fetch(0, kr, vr);
  stash(0, kr, vr);
  __syncthreads();
  for (int t = 0; t < n_tiles; ++t) {
    const bool more = t + 1 < n_tiles;  // the same for every wave of the workgroup
    if (more) fetch(t + 1, kr, vr);
    if (t < my_tiles) {
      scores(t & 1);
      softmax(t);
      weighted_values(t & 1);
    }
    // buffer (t + 1) & 1 was last read for tile t - 1, before the barrier that ended that round
    if (more) stash((t + 1) & 1, kr, vr);
    __syncthreads();
  }

  // ---- normalise and store -------------------------------------------------------
  float l_a, l_b;
  both_halves(l, l_a, l_b);
  const float lt = l_a + l_b;
  const float inv = lt > 0.f ? 1.f / lt : 0.f;
  if (my_q < C) {
    float *orow = reinterpret_cast<float *>(p.out) + (q_lo + my_q) * p.out_stride_token + (int64_t)h * HD;
#pragma unroll
    for (int ob = 0; ob < OB; ++ob) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = ob * 32 + 4 * hh + 8 * j;
        *reinterpret_cast<float4 *>(orow + d) = make_float4(o[ob][4 * j] * inv, o[ob][4 * j + 1] * inv,
                                                            o[ob][4 * j + 2] * inv, o[ob][4 * j + 3] * inv);
      }
    }
  }
}

template <bool SINGLE, bool MASK>
int launch_hd(const PrefillKP &kp, int hd, dim3 grid, hipStream_t stream) {
  switch (hd) {
    case 32:
      hipLaunchKernelGGL((paged_prefill_f32_kernel<32, SINGLE, MASK>), grid, dim3(kF32Threads), 0, stream, kp);
      break;
    case 64:
      hipLaunchKernelGGL((paged_prefill_f32_kernel<64, SINGLE, MASK>), grid, dim3(kF32Threads), 0, stream, kp);
      break;
    case 128:
      hipLaunchKernelGGL((paged_prefill_f32_kernel<128, SINGLE, MASK>), grid, dim3(kF32Threads), 0, stream, kp);
      break;
    default:
      return IC_ERR_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? IC_OK : IC_ERR_LAUNCH;
}

}  // namespace

int launch_paged_prefill_f32(PrefillKP kp, const PrefillArgs &a, hipStream_t stream) {
  kp.n_qtiles = (a.max_chunk_len + kF32BM - 1) / kF32BM;
  const int64_t wgs_x = (int64_t)kp.n_qtiles * a.hn;
  if (wgs_x > 0x7fffffff || a.n_seqs > 65535) return IC_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)wgs_x, (unsigned)a.n_seqs);
  const bool masked = a.mask != nullptr;
  // A one-column block table means one block per sequence, of any length.
  if (a.block_table_stride == 1)
    return masked ? launch_hd<true, true>(kp, a.hd, grid, stream) : launch_hd<true, false>(kp, a.hd, grid, stream);
  if (kp.block_size < 1) return IC_ERR_UNSUPPORTED;
  return masked ? launch_hd<false, true>(kp, a.hd, grid, stream) : launch_hd<false, false>(kp, a.hd, grid, stream);
}

}  // namespace prefill
}  // namespace ic
