// Paged decode: one query token per sequence against the block KV cache.
//
// What it computes is the reference's dense attention with sq = 1
// (ironcore/layers/attention.py:68-142) on the rows the block table names:
// scores = q.k * scale, softmax over the context, out = probs @ v, with query
// head h reading KV head h / G (attention.py:95-102).  Scores, softmax and the
// PV sum stay in fp32; only the result is rounded to the element type.
//
// HBM-bound streaming kernel (one pass over every visible K and V byte).
//
//  * grid = (split-K partition, kv head [x query sub-group], sequence).  A
//    workgroup owns `part_tokens` consecutive tokens of one (sequence, KV
//    head) and ALL G query heads that share that KV head, so each K/V byte
//    is fetched once per KV head, not once per query head.
//  * The partition's slice of the block table and the query group are staged
//    in LDS once; block ids are then wave-uniform scalars.
//  * A wave walks whole blocks.  One (block, kv head) tile is
//    block_size*hd elements; each lane fetches 16 bytes per load, so one load
//    instruction covers 1 KiB of consecutive tile bytes (64/LPR token rows,
//    LPR = lanes per row).  The next tile's loads are issued before the
//    current tile is consumed.
//  * q.k: v_dot2 on the packed pairs, then a DPP butterfly over the LPR lanes
//    that share a row.  Online softmax per lane group; p*v accumulates into
//    EPL fp32 registers per query head with no cross-lane traffic.
//  * Lane groups and waves are merged through LDS with a log-sum-exp
//    combine.  A sequence that fits one partition is finished here;
//    otherwise (m, l, acc) partials go to the workspace and the reduce kernel
//    below combines them.
//
// Algorithmic bytes per launch: sum_i ctx_i * 2 * gn * hd * elem (K and V,
// once per KV head) + q, out, block-table slice and context lengths.
#include "ic_device.h"
#include "ic_internal.h"
#include "../../include/ironcore_paged.h"

namespace ic {

namespace {

struct DecodeKP {
  const char *q;
  const char *k_pool;
  const char *v_pool;
  const int32_t *block_tables;
  const int32_t *context_lens;
  char *out;
  float *part_ml;
  float *part_acc;
  int64_t q_stride_seq;    // elements
  int64_t out_stride_seq;  // elements
  int64_t stride_block;    // elements
  int64_t stride_head;
  int64_t stride_token;
  int64_t bt_stride;
  int64_t num_blocks;
  int hn;
  int group;  // query heads per KV head
  int nsub;   // query sub-groups per KV head (ceil(group / GT))
  int max_ctx;
  int part_tokens;
  int n_parts;
  float scale_log2e;
};

constexpr float kNegInf = -__builtin_huge_valf();

// One WAVE owns one split-K partition of one (sequence, KV head): the waves
// of a workgroup never synchronise with each other, so a wave that finishes
// (or has no tokens) retires on its own and the CU always has other waves'
// loads in flight.  NW only sets how many partitions share a workgroup slot.
#ifndef IC_DECODE_NW
#define IC_DECODE_NW 4
#endif
#ifdef IC_DECODE_WAVES_PER_EU
#define IC_DECODE_OCC __attribute__((amdgpu_waves_per_eu(IC_DECODE_WAVES_PER_EU)))
#else
#define IC_DECODE_OCC
#endif

template <class E, int HD, int GT, int BS, int NW>
__global__ __launch_bounds__(NW *kWave) IC_DECODE_OCC void paged_decode_kernel(const DecodeKP p) {
  using T = typename E::type;
  constexpr int EPL = E::EPL;
  constexpr int ES = sizeof(T);
  constexpr int LPR = HD / EPL;     // lanes sharing one token row
  constexpr int RPL = kWave / LPR;  // token rows per load instruction
  constexpr int NLD = BS / RPL;     // load instructions per (block, head) tile
  static_assert(HD % EPL == 0 && kWave % LPR == 0 && BS % RPL == 0, "tile shape");

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int part = blockIdx.x * NW + wave;
  const int kvh = blockIdx.y / p.nsub;
  const int sub = blockIdx.y - kvh * p.nsub;
  const int seq = blockIdx.z;

  int ctx = p.context_lens[seq];
  ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
  const int tok_begin = part * p.part_tokens;
  if (tok_begin >= ctx) return;
  const int tok_end = (tok_begin + p.part_tokens < ctx) ? tok_begin + p.part_tokens : ctx;
  const int blk_begin = tok_begin / BS;
  const int nblk = (tok_end - tok_begin + BS - 1) / BS;  // <= 64 (checked on the host)
  const int n_parts_seq = (ctx + p.part_tokens - 1) / p.part_tokens;

  const int col = lane % LPR;
  const int rowg = lane / LPR;
  const int head0 = kvh * p.group + sub * GT;  // first query head of this wave
  const int heads_here = (p.group - sub * GT < GT) ? p.group - sub * GT : GT;

  // Lane i keeps the pool block of the partition's i-th block; the loop reads
  // it back as a wave-uniform scalar (v_readlane), so tile addresses are SALU
  // work and the table never sits on the load path again.
  int32_t my_block = 0;
  if (lane < nblk) {
    my_block = p.block_tables[seq * p.bt_stride + blk_begin + lane];
    // A corrupt table entry must not become an out-of-pool address.
    my_block = my_block < 0 ? 0 : my_block;
    my_block = (int64_t)my_block >= p.num_blocks ? (int32_t)(p.num_blocks - 1) : my_block;
  }

  Vec16 qreg[GT];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    qreg[g] = Vec16{{0u, 0u, 0u, 0u}};
    if (g < heads_here)
      qreg[g] = load16(p.q + (seq * p.q_stride_seq + (int64_t)(head0 + g) * HD + col * EPL) * ES);
  }

  uint32_t lane_off[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i)
    lane_off[i] = (uint32_t)(((i * RPL + rowg) * p.stride_token + col * EPL) * ES);

  float m[GT], l[GT], acc[GT][EPL];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = kNegInf;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
  }

  auto issue = [&](int j, Vec16 *kk, Vec16 *vv) {
    const int64_t phys = __builtin_amdgcn_readlane(my_block, j);
    const int64_t tile = (phys * p.stride_block + kvh * p.stride_head) * ES;
    const char *kb = p.k_pool + tile;
    const char *vb = p.v_pool + tile;
#pragma unroll
    for (int i = 0; i < NLD; ++i) kk[i] = load16(kb + lane_off[i]);
#pragma unroll
    for (int i = 0; i < NLD; ++i) vv[i] = load16(vb + lane_off[i]);
    // Keep the loads ahead of the arithmetic that follows in program order:
    // the scheduler would otherwise sink them below the current tile's work
    // and shorten the prefetch distance.
    __builtin_amdgcn_sched_barrier(0);
  };

  // `last` marks the partition's final tile, the only one that can be partly
  // filled; every other tile skips the validity test.
  auto consume = [&](int j, Vec16 *kk, Vec16 *vv, bool last) {
    const int tok0 = tok_begin + j * BS;
    float s[GT][NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        float d = E::dot(kk[i], qreg[g], 0.f);
        s[g][i] = group_sum<LPR>(d) * p.scale_log2e;
      }
    }
    if (last && tok0 + BS > tok_end) {  // partly filled block: hide the unused slots
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        if (tok0 + i * RPL + rowg >= tok_end) {
#pragma unroll
          for (int g = 0; g < GT; ++g) s[g][i] = kNegInf;
          vv[i] = Vec16{{0u, 0u, 0u, 0u}};
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
  };

  {
    // Two register tiles in ping-pong.  The steady-state loop issues the next
    // tile's loads unconditionally, so the wait before a tile is consumed
    // covers that tile only and the prefetch stays in flight behind it.
    Vec16 ka[NLD], va[NLD], kb[NLD], vb[NLD];
    int j = 0;
    issue(0, ka, va);
    for (; j + 2 < nblk; j += 2) {
      issue(j + 1, kb, vb);
      consume(j, ka, va, false);
      issue(j + 2, ka, va);
      consume(j + 1, kb, vb, false);
    }
    if (j + 2 == nblk) {
      issue(j + 1, kb, vb);
      consume(j, ka, va, false);
      consume(j + 1, kb, vb, true);
    } else {
      consume(j, ka, va, true);
    }
  }

  // ---- merge the RPL row groups of this wave (log-sum-exp combine) -----------
  __shared__ __attribute__((aligned(16))) float s_acc[NW][RPL][GT][HD];
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
  }
  // Only this wave reads what it wrote: a wave-level LDS fence is enough.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    if (g >= heads_here) break;
    const int h = head0 + g;
    const int64_t slot = ((int64_t)seq * p.hn + h) * p.n_parts + part;
#pragma unroll
    for (int d = lane; d < HD; d += kWave) {
      float a = 0.f;
#pragma unroll
      for (int r = 0; r < RPL; ++r) a += s_acc[wave][r][g][d];
      if (n_parts_seq == 1)
        reinterpret_cast<T *>(p.out)[seq * p.out_stride_seq + (int64_t)h * HD + d] = E::narrow(a / lsum[g]);
      else
        p.part_acc[slot * HD + d] = a;
    }
    if (n_parts_seq != 1 && lane == 0) {
      p.part_ml[slot * 2] = mall[g];
      p.part_ml[slot * 2 + 1] = lsum[g];
    }
  }
}

// Combine the split-K partials of one (sequence, query head).
// grid = (hn, n_seqs), HD threads.  Traffic is n_parts*(hd+2)*4 bytes per
// head, three orders of magnitude below the K/V stream.
template <class E, int HD>
__global__ __launch_bounds__(HD) void paged_decode_reduce_kernel(const DecodeKP p) {
  using T = typename E::type;
  const int h = blockIdx.x;
  const int seq = blockIdx.y;
  const int d = threadIdx.x;
  int ctx = p.context_lens[seq];
  ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
  T *o = reinterpret_cast<T *>(p.out) + seq * p.out_stride_seq + (int64_t)h * HD + d;
  if (ctx <= 0) {
    *o = E::narrow(0.f);
    return;
  }
  const int np = (ctx + p.part_tokens - 1) / p.part_tokens;
  if (np == 1) return;  // finished by the main kernel
  const int64_t slot0 = ((int64_t)seq * p.hn + h) * p.n_parts;
  float mx = kNegInf;
  for (int i = 0; i < np; ++i) mx = fmaxf(mx, p.part_ml[(slot0 + i) * 2]);
  float lsum = 0.f, a = 0.f;
  for (int i = 0; i < np; ++i) {
    const float w = __builtin_amdgcn_exp2f(p.part_ml[(slot0 + i) * 2] - mx);
    lsum = __builtin_fmaf(p.part_ml[(slot0 + i) * 2 + 1], w, lsum);
    a = __builtin_fmaf(p.part_acc[(slot0 + i) * HD + d], w, a);
  }
  *o = E::narrow(a / lsum);
}

template <class E, int HD, int GT>
int launch_typed(const DecodeKP &kp, int gn, int n_seqs, hipStream_t stream) {
  constexpr int BS = 16;
  constexpr int NW = IC_DECODE_NW;
  dim3 grid((kp.n_parts + NW - 1) / NW, gn * kp.nsub, n_seqs);
  hipLaunchKernelGGL((paged_decode_kernel<E, HD, GT, BS, NW>), grid, dim3(NW * kWave), 0, stream, kp);
  hipLaunchKernelGGL((paged_decode_reduce_kernel<E, HD>), dim3(kp.hn, n_seqs), dim3(HD), 0, stream, kp);
  return hipGetLastError() == hipSuccess ? IC_OK : IC_ERR_LAUNCH;
}

template <class E, int HD>
int launch_group(DecodeKP &kp, int gn, int n_seqs, hipStream_t stream) {
  const int G = kp.group;
  const int gt = G <= 8 ? G : 8;
  kp.nsub = (G + gt - 1) / gt;
  switch (gt) {
    case 1: return launch_typed<E, HD, 1>(kp, gn, n_seqs, stream);
    case 2: return launch_typed<E, HD, 2>(kp, gn, n_seqs, stream);
    case 3: return launch_typed<E, HD, 3>(kp, gn, n_seqs, stream);
    case 4: return launch_typed<E, HD, 4>(kp, gn, n_seqs, stream);
    case 5: return launch_typed<E, HD, 5>(kp, gn, n_seqs, stream);
    case 6: return launch_typed<E, HD, 6>(kp, gn, n_seqs, stream);
    case 7: return launch_typed<E, HD, 7>(kp, gn, n_seqs, stream);
    default: return launch_typed<E, HD, 8>(kp, gn, n_seqs, stream);
  }
}

template <class E>
int launch_hd(DecodeKP &kp, int hd, int gn, int n_seqs, hipStream_t stream) {
  switch (hd) {
    case 64: return launch_group<E, 64>(kp, gn, n_seqs, stream);
    case 128: return launch_group<E, 128>(kp, gn, n_seqs, stream);
    default: return IC_ERR_UNSUPPORTED;
  }
}

}  // namespace

int launch_paged_decode(const DecodeArgs &a, hipStream_t stream) {
  if (a.pool.block_size != 16) return IC_ERR_UNSUPPORTED;
  DecodeKP kp;
  kp.q = (const char *)a.q;
  kp.k_pool = (const char *)a.k_pool;
  kp.v_pool = (const char *)a.v_pool;
  kp.block_tables = a.block_tables;
  kp.context_lens = a.context_lens;
  kp.out = (char *)a.out;
  kp.part_ml = a.part_ml;
  kp.part_acc = a.part_acc;
  kp.q_stride_seq = a.q_stride_seq;
  kp.out_stride_seq = a.out_stride_seq;
  kp.stride_block = a.pool.stride_block;
  kp.stride_head = a.pool.stride_head;
  kp.stride_token = a.pool.stride_token;
  kp.bt_stride = a.block_table_stride;
  kp.num_blocks = a.pool.num_blocks;
  kp.hn = a.hn;
  kp.group = a.hn / a.gn;
  kp.nsub = 1;
  kp.max_ctx = a.max_context_len;
  kp.part_tokens = a.part_tokens;
  kp.n_parts = a.n_parts;
  kp.scale_log2e = a.scale * 1.4426950408889634f;
  switch (a.dtype) {
    case IC_DTYPE_BF16: return launch_hd<Bf16>(kp, a.hd, a.gn, a.n_seqs, stream);
    case IC_DTYPE_F16: return launch_hd<F16>(kp, a.hd, a.gn, a.n_seqs, stream);
    case IC_DTYPE_F32: return launch_hd<F32>(kp, a.hd, a.gn, a.n_seqs, stream);
    default: return IC_ERR_UNSUPPORTED;
  }
}

}  // namespace ic
