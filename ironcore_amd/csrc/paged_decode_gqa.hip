// Paged decode for grouped-query attention (several query heads per KV head).
//
// Same result, same balanced split-K bookkeeping, same partial format and
// reduce pass as paged_decode.hip; what changes is how a tile's arithmetic is
// laid over the lanes, because with G query heads per K/V byte the
// single-head mapping runs out of VALU issue slots long before it runs out
// of HBM bandwidth.  Per 16-token tile and G heads:
//
//  * q.k: ONE TOKEN PER QUAD.  Lane l holds a quarter (hd/4 dims) of token
//    l/4's K row; the G query rows sit in LDS and are read as broadcasts.
//    A score needs 2 DPP adds (quad_perm) instead of a 16-lane butterfly, and
//    each lane ends with the G scores of ONE token, so the tile costs G
//    v_exp per lane instead of 4 G.
//  * Running maximum: kept per head as a wave-uniform reference and only
//    moved when some score exceeds it by more than 2^5; until then no
//    cross-lane reduction and no rescale of the accumulators happens at all
//    (for iid scores that is the first tile of a segment and almost never
//    again).  Probabilities stay <= 32 and the sum is exact in fp32.
//  * p.v: probabilities go through a 256-byte LDS slab as packed 16-bit pairs
//    (the reference rounds them to the element type too), V stays in the
//    coalesced row mapping (16 bytes per lane), pairs of tokens are packed
//    with v_perm_b32 and each head costs hd/8 v_dot2 per lane per 4 tokens.
//
// About 45 VALU issue slots per head per tile instead of 110.
#include "decode_common.h"
#include "../../include/ironcore_paged.h"

namespace ic {
namespace decode {

namespace {

constexpr float kLazyMaxSlack = 5.0f;  // log2 units

__device__ __forceinline__ float dpp_max(float x, float y) { return fmaxf(x, y); }

// max / sum over the 16 token slots of a tile: lanes l/4 (quads hold copies).
__device__ __forceinline__ float token_max(float x) {
  x = fmaxf(x, dpp_f32<kDppRowRor4>(x));
  x = fmaxf(x, dpp_f32<kDppRowRor8>(x));
  x = fmaxf(x, __shfl_xor(x, 16, kWave));
  x = fmaxf(x, __shfl_xor(x, 32, kWave));
  return x;
}
__device__ __forceinline__ float token_sum(float x) {
  x += dpp_f32<kDppRowRor4>(x);
  x += dpp_f32<kDppRowRor8>(x);
  x += __shfl_xor(x, 16, kWave);
  x += __shfl_xor(x, 32, kWave);
  return x;
}

#ifdef IC_GQA_WAVES_PER_EU
#define IC_GQA_OCC __attribute__((amdgpu_waves_per_eu(IC_GQA_WAVES_PER_EU)))
#else
#define IC_GQA_OCC
#endif

template <class E, int HD, int GT, int BS, int NW>
__global__ __launch_bounds__(NW *kWave) IC_GQA_OCC void paged_decode_gqa_kernel(const DecodeKP p) {
  using T = typename E::type;
  static_assert(sizeof(T) == 2, "16-bit element types only");
  constexpr int ES = 2;
  constexpr int DPL = HD / 4;       // K side: dims per lane (a quad covers one token row)
  constexpr int NK = DPL / 8;       // K side: 16-byte loads per lane per tile
  constexpr int LPR = HD / 8;       // V side: lanes sharing one token row
  constexpr int RPL = kWave / LPR;  // V side: token rows per load instruction
  constexpr int NLD = BS / RPL;     // V side: loads per tile = tokens per lane
  constexpr int SW = 4;
  constexpr int NQ = (GT * HD / 8 + kWave - 1) / kWave;  // 16-byte q chunks per lane
  static_assert(BS == 16 && (NLD == 2 || NLD == 4), "tile shape");

  __shared__ __attribute__((aligned(16))) T s_q[NW][GT * HD];
  __shared__ __attribute__((aligned(8))) T s_p[NW][RPL][GT][NLD];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int tq = lane >> 2;         // K side: token of this lane's quad
  const int qc = lane & 3;          // K side: which quarter of the row
  const int col = lane % LPR;       // V side
  const int rowg = lane / LPR;      // V side

  const int64_t wid = (int64_t)blockIdx.x * NW + wave;
  int64_t left;
  TileCursor c;
  if (!locate_chunk<BS>(p, lane, wid, left, c)) return;
  TileCursor walk = c;
  TileCursor peek = c;
  next_pair<BS>(p, peek);
  int seg_blk0 = c.blk;

  uint32_t k_off[NK], v_off[NLD];
#pragma unroll
  for (int j = 0; j < NK; ++j) k_off[j] = (uint32_t)((tq * p.stride_token + qc * DPL + j * 8) * ES);
#pragma unroll
  for (int i = 0; i < NLD; ++i) v_off[i] = (uint32_t)(((i * RPL + rowg) * p.stride_token + col * 8) * ES);

  // query rows of a pair: global -> registers (a segment ahead) -> LDS
  auto fetch_q = [&](const TileCursor &tc, Vec16 *qq) {
    const int kvh = tc.pair / p.nsub;
    const int sub = tc.pair - kvh * p.nsub;
    const int head0 = kvh * p.group + sub * GT;
    const int heads = (p.group - sub * GT < GT) ? p.group - sub * GT : GT;
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int chunk = u * kWave + lane;  // 16-byte chunk of the [GT][HD] block
      qq[u] = Vec16{{0u, 0u, 0u, 0u}};
      if (chunk * 8 < heads * HD && tc.seq < p.n_seqs)
        qq[u] = load16(p.q + (tc.seq * p.q_stride_seq + (int64_t)head0 * HD + chunk * 8) * ES);
    }
  };
  auto park_q = [&](const Vec16 *qq) {
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int chunk = u * kWave + lane;
      if (chunk * 8 < GT * HD) store16(&s_q[wave][chunk * 8], qq[u]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  Vec16 qnext[NQ];
  fetch_q(c, qnext);
  park_q(qnext);
  fetch_q(peek, qnext);

  float m[GT], l[GT], acc[GT][8];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = kNegInf;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
  }

  auto finish_segment = [&]() {
    const int kvh = c.pair / p.nsub;
    const int sub = c.pair - kvh * p.nsub;
    const int head0 = kvh * p.group + sub * GT;
    const int heads = (p.group - sub * GT < GT) ? p.group - sub * GT : GT;
    const bool whole_pair = (seg_blk0 == 0 && c.blk == c.nb);
    const int64_t partial = wid + (int64_t)c.seq * p.pairs_per_seq + c.pair;
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (g >= heads) break;
      const float lsum = token_sum(l[g]);
      // All V-side rows share the reference maximum: their accumulators just add.
      float a[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        a[e] = acc[g][e];
#pragma unroll
        for (int step = LPR; step < kWave; step <<= 1) a[e] += __shfl_xor(a[e], step, kWave);
      }
      const int h = head0 + g;
      if (rowg == 0) {  // one row writes dims col*8 .. col*8+7
        if (whole_pair) {
          const float inv = 1.f / lsum;
          T *o = reinterpret_cast<T *>(p.out) + c.seq * p.out_stride_seq + (int64_t)h * HD + col * 8;
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = E::narrow(a[e] * inv);
        } else {
          float *o = p.part_acc + (partial * GT + g) * HD + col * 8;
          *reinterpret_cast<float4 *>(o) = make_float4(a[0], a[1], a[2], a[3]);
          *reinterpret_cast<float4 *>(o + 4) = make_float4(a[4], a[5], a[6], a[7]);
        }
      }
      if (!whole_pair && lane == 0) {
        p.part_ml[(partial * GT + g) * 2] = m[g];
        p.part_ml[(partial * GT + g) * 2 + 1] = lsum;
      }
    }
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      m[g] = kNegInf;
      l[g] = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    }
    if (left > 0) {
      c = peek;
      seg_blk0 = 0;
      park_q(qnext);
      next_pair<BS>(p, peek);
      fetch_q(peek, qnext);
    }
  };

  auto consume = [&](Vec16 *kk, Vec16 *vv) {
    // ---- scores: this lane's quad owns token tq of the tile ----------------------
    float s[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      float d = 0.f;
#pragma unroll
      for (int j = 0; j < NK; ++j) d = E::dot(kk[j], load16(&s_q[wave][g * HD + qc * DPL + j * 8]), d);
      d += dpp_f32<kDppQuadXor1>(d);
      d += dpp_f32<kDppQuadXor2>(d);
      s[g] = d * p.scale_log2e;
    }
    if (c.blk == c.nb - 1) {  // the sequence's last block may be partly filled
      int ctx = p.context_lens[c.seq];
      ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
      const int tok0 = c.blk * BS;
      if (tok0 + BS > ctx) {
        if (tok0 + tq >= ctx) {
#pragma unroll
          for (int g = 0; g < GT; ++g) s[g] = kNegInf;
        }
#pragma unroll
        for (int i = 0; i < NLD; ++i)
          if (tok0 + i * RPL + rowg >= ctx) vv[i] = Vec16{{0u, 0u, 0u, 0u}};
      }
    }
    // ---- lazy running maximum --------------------------------------------------
    bool exceed = false;
#pragma unroll
    for (int g = 0; g < GT; ++g) exceed |= s[g] > m[g] + kLazyMaxSlack;
    if (__any(exceed)) {  // wave-uniform, rare after a segment's first tile
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        const float m_new = fmaxf(m[g], token_max(s[g]));
        const float alpha = (m[g] == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m[g] - m_new);
        l[g] *= alpha;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] *= alpha;
        m[g] = m_new;
      }
    }
    // ---- probabilities -> LDS as 16-bit, grouped for the V-side rows -------------
    float pr[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      const float ms = (m[g] == kNegInf) ? 0.f : m[g];
      pr[g] = __builtin_amdgcn_exp2f(s[g] - ms);
      l[g] += pr[g];
    }
#pragma unroll
    for (int k = 0; k * 4 < GT; ++k) {  // lane qc writes heads qc, qc+4, ...
      const float a0 = pr[4 * k];
      const float a1 = 4 * k + 1 < GT ? pr[4 * k + 1] : 0.f;
      const float a2 = 4 * k + 2 < GT ? pr[4 * k + 2] : 0.f;
      const float a3 = 4 * k + 3 < GT ? pr[4 * k + 3] : 0.f;
      const float lo = (qc & 1) ? a1 : a0;
      const float hi = (qc & 1) ? a3 : a2;
      const float mine = (qc & 2) ? hi : lo;
      if (4 * k + qc < GT) s_p[wave][tq % RPL][4 * k + qc][tq / RPL] = E::narrow(mine);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // ---- p.v: pack token pairs, one v_dot2 per (head, dim, pair) ------------------
    // vv[i] holds token (i*RPL + rowg), dims col*8 .. col*8+7 as 4 packed dwords.
    uint32_t lo01[4], hi01[4], lo23[4], hi23[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      lo01[k] = __builtin_amdgcn_perm(vv[1].w[k], vv[0].w[k], 0x05040100u);
      hi01[k] = __builtin_amdgcn_perm(vv[1].w[k], vv[0].w[k], 0x07060302u);
      if (NLD == 4) {
        lo23[k] = __builtin_amdgcn_perm(vv[3 % NLD].w[k], vv[2 % NLD].w[k], 0x05040100u);
        hi23[k] = __builtin_amdgcn_perm(vv[3 % NLD].w[k], vv[2 % NLD].w[k], 0x07060302u);
      }
    }
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      uint32_t p01, p23 = 0;
      if (NLD == 4) {
        const uint2 pp = *reinterpret_cast<const uint2 *>(&s_p[wave][rowg][g][0]);
        p01 = pp.x;
        p23 = pp.y;
      } else {
        p01 = *reinterpret_cast<const uint32_t *>(&s_p[wave][rowg][g][0]);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc[g][2 * k] = E::dot2(lo01[k], p01, acc[g][2 * k]);
        acc[g][2 * k + 1] = E::dot2(hi01[k], p01, acc[g][2 * k + 1]);
        if (NLD == 4) {
          acc[g][2 * k] = E::dot2(lo23[k], p23, acc[g][2 * k]);
          acc[g][2 * k + 1] = E::dot2(hi23[k], p23, acc[g][2 * k + 1]);
        }
      }
    }
    // the slab is rewritten by the next tile
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    ++c.blk;
    --left;
    if (c.blk == c.nb || left == 0) finish_segment();
  };

  while (left > 0) {
    const int n_win = left < kWave * SW ? (int)left : kWave * SW;
    uint32_t off_lo[SW], off_hi[SW];
    gather_window<BS, SW, ES>(p, lane, n_win, walk, off_lo, off_hi);

    auto issue = [&](int i, Vec16 *kk, Vec16 *vv) {
      const int64_t tile = window_tile_offset(off_lo, off_hi, i);
      const char *kb = p.k_pool + tile;
      const char *vb = p.v_pool + tile;
#pragma unroll
      for (int j = 0; j < NK; ++j) kk[j] = load16(kb + k_off[j]);
#pragma unroll
      for (int j = 0; j < NLD; ++j) vv[j] = load16(vb + v_off[j]);
      __builtin_amdgcn_sched_barrier(0);
    };

    Vec16 ka[NK], va[NLD], kb[NK], vb[NLD];
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

template <class E, int HD, int GT>
bool launch_one(DecodeKP &kp, hipStream_t stream) {
  constexpr int BS = 16;
  constexpr int NW = kDecodeWavesPerWorkgroup;
  static const int per_cu = [] {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, paged_decode_gqa_kernel<E, HD, GT, BS, NW>,
                                                     NW * kWave, 0) != hipSuccess || n < 1)
      n = 1;
    return n;
  }();
  int wgs = per_cu * device_cu_count();
  if (wgs * NW > kMaxDecodeWaves) wgs = kMaxDecodeWaves / NW;
  kp.n_waves = wgs * NW;
  hipLaunchKernelGGL((paged_decode_gqa_kernel<E, HD, GT, BS, NW>), dim3(wgs), dim3(NW * kWave), 0, stream, kp);
  return true;
}

template <class E, int HD>
bool launch_gt(DecodeKP &kp, int gt, hipStream_t stream) {
  switch (gt) {
    case 2: return launch_one<E, HD, 2>(kp, stream);
    case 3: return launch_one<E, HD, 3>(kp, stream);
    case 4: return launch_one<E, HD, 4>(kp, stream);
    case 5: return launch_one<E, HD, 5>(kp, stream);
    case 6: return launch_one<E, HD, 6>(kp, stream);
    case 7: return launch_one<E, HD, 7>(kp, stream);
    case 8: return launch_one<E, HD, 8>(kp, stream);
    default: return false;
  }
}

template <class E>
bool launch_hd(DecodeKP &kp, int hd, int gt, hipStream_t stream) {
  switch (hd) {
    case 64: return launch_gt<E, 64>(kp, gt, stream);
    case 128: return launch_gt<E, 128>(kp, gt, stream);
    default: return false;
  }
}

}  // namespace

bool launch_decode_gqa_main(DecodeKP &kp, int dtype, int hd, int gt, hipStream_t stream) {
  switch (dtype) {
    case IC_DTYPE_BF16: return launch_hd<Bf16>(kp, hd, gt, stream);
    case IC_DTYPE_F16: return launch_hd<F16>(kp, hd, gt, stream);
    default: return false;
  }
}

}  // namespace decode
}  // namespace ic
