// Paged decode main kernel for 16-bit element types (bf16, fp16), on the
// matrix cores, for any number G of query heads per KV head (up to 16 matrix
// columns per wave).
//
// Same result, same balanced split-K bookkeeping, same partial format and
// reduce pass as paged_decode.hip.  What changes is the arithmetic of a tile:
// with G query heads per K/V byte the vector ALU runs out of issue slots long
// before HBM runs out of bandwidth, so both products of a 16-token tile go to
// MFMA with the (up to 16) query heads of the pair as one matrix dimension.
//
//  * K and V tiles are fetched in memory order: a 16-lane group reads 256
//    contiguous bytes of one token row.  (Fetching K straight into the matrix
//    layout, one 16-byte piece of each of 16 rows per group, costs the L1
//    eight times the tag look-ups and caps a cache-resident tile at 1.0 us per
//    wave instead of 0.6.)  K then takes one hop through a wave-private LDS
//    tile, rows padded by 16 bytes, and comes back in the matrix layout.
//  * S = K . Q^T   (v_mfma_f32_16x16x32, hd/32 of them).  A = the K tile:
//    lane l supplies row l%16 and the 8 dims 32j + 8(l/16) .. +7.  B = the
//    query rows, held in registers for the whole segment: lane l supplies
//    head l%16 (zero beyond the pair's heads), same dims.  The result leaves
//    lane l with the scores of head l%16 for the four S rows 4(l/16) .. +3.
//  * S row i is token (i/4) + 4(i%4) of the tile (a lane just reads that
//    token's K row back from LDS), so lane l owns tokens kg, kg+4, kg+8, kg+12
//    (kg = l/16): exactly the four k-elements lane l must supply for matrix A
//    of the next product.  exp2 and the 16-bit rounding (the reference rounds
//    the probabilities to the element type too, attention.py:124-134) happen
//    in place.
//  * O += P . V    (v_mfma_f32_16x16x16, one per dim owned by a lane).  B = V:
//    lane l loads dims (l%16)*hd/16 .. of tokens kg + 4i and packs token pairs
//    with v_perm_b32; MFMA e covers dim (l%16)*hd/16 + e.  The accumulators
//    leave lane l with heads 4kg .. 4kg+3 of those dims.
//  * Running maximum: a per-head reference that only moves when some score
//    exceeds it by more than 2^5 (wave-uniform test); until then there is no
//    cross-lane reduction and no rescale.  Row sums stay per lane and are
//    folded once per segment.
//
// Per tile and wave: hd/32 + hd/16 MFMAs, about 70 vector instructions and
// 2 * hd/32 LDS accesses, whatever G is: about 0.6 us when the tile is in the
// cache, which leaves the kernel bound by HBM for any pool that is not.
#include <atomic>
#include <type_traits>

#include "decode_common.h"
#include "../../include/ironcore_paged.h"

namespace ic {
namespace decode {

namespace {

std::atomic<long long> g_occupancy_queries{0};  // runtime occupancy queries made so far (a diagnostic)

constexpr float kLazyMaxSlack = 5.0f;  // log2 units
constexpr int kLongRowTokens = 1024;      // longest context from which one workgroup per CU is launched
constexpr int kVeryLongRowTokens = 4096;  // ... and from which one CU in eight is left out

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;

struct Pair32 {
  uint32_t lo, hi;
};

struct MfmaBf16 : Bf16 {
  static __device__ __forceinline__ f32x4_t qk(const Vec16 &a, const Vec16 &b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t pv(const Pair32 &a, const Pair32 &b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a),
                                                     __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    const bf16x2_t v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};

struct MfmaF16 : F16 {
  static __device__ __forceinline__ f32x4_t qk(const Vec16 &a, const Vec16 &b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t pv(const Pair32 &a, const Pair32 &b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a),
                                                 __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    const f16x2_t v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};

// VW dwords (2*VW elements) of one V row.
template <int VW>
struct VChunk {
  uint32_t w[VW];
};
template <int VW>
__device__ __forceinline__ VChunk<VW> load_v(const void *p);
template <>
__device__ __forceinline__ VChunk<4> load_v<4>(const void *p) {
  const Vec16 v = load16(p);
  return VChunk<4>{{v.w[0], v.w[1], v.w[2], v.w[3]}};
}
template <>
__device__ __forceinline__ VChunk<2> load_v<2>(const void *p) {
  const uint2 v = *reinterpret_cast<const uint2 *>(p);
  return VChunk<2>{{v.x, v.y}};
}
template <>
__device__ __forceinline__ VChunk<1> load_v<1>(const void *p) {
  return VChunk<1>{{*reinterpret_cast<const uint32_t *>(p)}};
}

// With shared-prefix cohorts the kernel runs two phases (see DecodeKP); every
// other workgroup takes them in the opposite order, so that the LDS-fed
// shared phase and the HBM-bound own phase overlap in time.
// PLAN: the rows' prefix sums are laid out in LDS once per workgroup
// (build_plan); otherwise (batches too long for LDS) every wave scans the rows.
// COOP: a unit of the shared phase is the whole workgroup, and its waves pass
// the shared tiles to each other through LDS: per round of NW tiles every wave
// fetches ONE of them from memory (a full round ahead) and leaves it in its
// slot of an LDS ring, and all waves then read each of the NW tiles back, K
// in the matrix layout, V lane for lane.  A shared tile so crosses the memory
// system once per workgroup instead of once per wave.
template <class E, int HD, int BS, int NW, bool PLAN, bool COOP>
// Two waves per SIMD is the design point (two 8 KiB tiles in flight each).
__global__ __launch_bounds__(NW *kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
void paged_decode_mfma_kernel(const DecodeKP p) {
  constexpr int NCB = 1;  // 16-column blocks of the query matrix a wave carries
  using T = typename E::type;
  constexpr int ES = 2;
  constexpr int NK = HD / 32;  // q.k MFMAs = 16-byte K pieces per lane per tile
  constexpr int VE = HD / 16;  // V dims per lane = p.v MFMAs per tile
  constexpr int VW = VE / 2;   // dwords per V load
  constexpr int NT = 4;        // tokens per lane on the V side
  constexpr int SW = 4;
  static_assert(sizeof(T) == 2 && BS == 16 && (VW == 1 || VW == 2 || VW == 4), "tile shape");

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int n = lane & 15;   // matrix column: head (q.k) or dim group (p.v)
  const int kg = lane >> 4;  // this lane's tokens are kg, kg+4, kg+8, kg+12

  const int64_t wave_id = (int64_t)xcd_major_workgroup() * NW + wave;
  const bool cohorts = p.cohort_size > 1;
  typedef const __attribute__((address_space(4))) int32_t *ScalarPtr;  // read through the scalar cache
  const ScalarPtr ctx_lens = (ScalarPtr)(unsigned long long)p.context_lens;
  extern __shared__ int plan_mem[];
  PlanLds plan;
  if constexpr (PLAN) {
    plan = plan_carve(plan_mem, p);
    build_plan<BS, NW * kWave>(p, plan, wave_id < NW);
  }
  // behind the plan: the ring of the cooperative shared phase (NW slots of one K and one V
  // tile), then one K staging tile per wave
  char *lds_tiles = reinterpret_cast<char *>(plan_mem + (PLAN ? ring_offset_ints(p.n_seqs, p.n_cohorts) : 0));
  constexpr int kSlotBytes = 16 * (HD * 2 + 16) + (NT * VW / 4) * kWave * 16;  // padded K rows, then V lane by lane
  char *xpose = lds_tiles + (COOP ? NW * kSlotBytes : 0) + wave * (16 * (HD * 2 + 16));  // this wave's K staging
  const int n_phases = cohorts ? 2 : 1;
  for (int phase = 0; phase < n_phases; ++phase) {
  // 0: rows are sequences, a share per wave; 1: rows are cohorts' shared tiles, a share per unit
  // (workgroups of one XCD go to its CUs in turn: neighbours on a CU and across CUs alternate)
  const int order = ((blockIdx.x >> 3) ^ (blockIdx.x >> 8)) & 1;
  const int shared = cohorts ? (phase ^ order) : 0;
  const int64_t wid = shared ? wave_id >> p.unit_shift : wave_id;
  const int cb_unit = shared ? (int)(wave_id & ((1 << p.unit_shift) - 1)) : 0;  // this wave's place in its unit
  // the phase's rows
  using Rows = typename std::conditional<PLAN, PlannedRows, GlobalRows<BS>>::type;
  const Rows rows = [&] {
    if constexpr (PLAN)
      return PlannedRows{shared ? plan.cum_sh : plan.cum_own, plan.eff_sh, phase_rows(p, shared), p.cohort_size,
                         shared};
    else
      return GlobalRows<BS>{p, shared};
  }();
  int64_t left64;
  TileCursor c;
  bool has;
  if constexpr (PLAN)
    has = locate_planned(p, rows, phase_units(p, shared), lane, wid, left64, c);
  else
    has = locate_chunk<BS>(p, lane, shared, wid, left64, c);
  if (!has) continue;
  // wave-uniform by construction; say so, so the bookkeeping is scalar work
  c.pair = __builtin_amdgcn_readfirstlane(c.pair);
  c.blk = __builtin_amdgcn_readfirstlane(c.blk);
  int left = __builtin_amdgcn_readfirstlane((int)left64);
  TileCursor walk = c;
  int seg_blk0 = c.blk;
  const int COLS = p.gt;  // columns per partial slot

  // K side: S row n is token (n/4) + 4(n%4).
  const int tok_k = (n >> 2) + 4 * (n & 3);
  uint32_t k_off[NK], v_off[NT];
  // K: piece f = 64j + lane of the tile in memory order is fetched by load j, written to LDS
  // at kst_off[j] and read back in the matrix layout at kld_off + 64j.
  constexpr int CPT = HD * ES / 16;     // 16-byte pieces per K row
  constexpr int KPITCH = HD * ES + 16;  // LDS row pitch: rows 4 banks apart, reads and writes conflict-free
  uint32_t kst_off[NK];
#pragma unroll
  for (int j = 0; j < NK; ++j) {
    const int f = j * kWave + lane;
    k_off[j] = (uint32_t)((f / CPT) * p.stride_token * ES + (f % CPT) * 16);
    kst_off[j] = (uint32_t)((f / CPT) * KPITCH + (f % CPT) * 16);
  }
  const uint32_t kld_off = (uint32_t)(tok_k * KPITCH + kg * 16);
#pragma unroll
  for (int i = 0; i < NT; ++i) v_off[i] = (uint32_t)(((kg + 4 * i) * p.stride_token + n * VE) * ES);

  // Shared phase: matrix column col is (member col / group of this wave's
  // members, head col % group); a lane's columns never change, so split them
  // once: (member << 16) | head.
  auto split = [&](int col) {
    if (!cohorts) return col;
    const int u = col / p.group;
    return (u << 16) | (col - u * p.group);
  };
  int ug_q[NCB], ug_o[NCB][4];  // this lane's column of q.k; its four columns of the accumulators
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    ug_q[cb] = split(cb * 16 + n);
#pragma unroll
    for (int r = 0; r < 4; ++r) ug_o[cb][r] = split(cb * 16 + 4 * kg + r);
  }
  // Wave-uniform facts about a segment's row and pair.
  struct Segment {
    int head0;   // first query head of the pair
    int heads;   // query heads of the pair in this segment (own phase)
    int seq0;    // the row's sequence; shared phase: this wave's first member
    int seq_end; // shared phase: one past the cohort's last sequence
  };
  auto segment_of = [&](const TileCursor &tc) {
    const int kvh = tc.pair / p.nsub;
    if (!shared) {
      const int sub = tc.pair - kvh * p.nsub;
      const int rest = p.group - sub * COLS;
      return Segment{kvh * p.group + sub * COLS, rest < COLS ? rest : COLS, tc.seq, 0};
    }
    const int first = tc.seq * p.cohort_size;
    const int end = first + p.cohort_size < p.n_seqs ? first + p.cohort_size : p.n_seqs;
    return Segment{kvh * p.group, p.group, first + cb_unit * p.spw, end};
  };
  Segment seg = segment_of(c);
  // Which (sequence, query head) a matrix column of the current segment is;
  // seq < 0 marks an unused column.
  auto column = [&](int col, int ug, int &seq, int &head) {
    if (!shared) {
      seq = col < seg.heads ? seg.seq0 : -1;
      head = seg.head0 + col;
    } else {
      const int u = ug >> 16;
      const int sq = seg.seq0 + u;
      seq = (u < p.spw && sq < seg.seq_end) ? sq : -1;
      head = seg.head0 + (ug & 0xffff);
    }
  };
  // matrix B of q.k: column n of each block, dims 32j + 8kg .. +7
  Vec16 qreg[NCB][NK];
  auto fetch_q = [&]() {
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      int seq, head;
      column(cb * 16 + n, ug_q[cb], seq, head);
#pragma unroll
      for (int j = 0; j < NK; ++j) {
        qreg[cb][j] = Vec16{{0u, 0u, 0u, 0u}};
        if (seq >= 0)
          qreg[cb][j] = load16(p.q + (seq * p.q_stride_seq + (int64_t)head * HD + 32 * j + 8 * kg) * ES);
      }
    }
  };
  fetch_q();

  float m[NCB], l[NCB];  // per column n: reference maximum (same in all kg groups), this lane's row sum
  f32x4_t acc[NCB][VE];  // acc[cb][e][r]: column 16cb + 4kg + r, dim n*VE + e
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    m[cb] = kNegInf;
    l[cb] = 0.f;
#pragma unroll
    for (int e = 0; e < VE; ++e) acc[cb][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  auto finish_segment = [&]() {
    // A segment that is all a sequence has (its whole row, and no shared
    // tiles besides) writes the output rows; anything else leaves a partial.
    const bool sole = !shared && c.first == 0;
    const bool whole_pair = sole && seg_blk0 == 0 && c.blk == c.nb;
    int64_t partial = wid + (int64_t)c.seq * p.pairs_per_seq + c.pair;
    if (shared) partial = p.shared_slot0 + (partial << p.unit_shift) + cb_unit;
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      float lsum = l[cb];
      lsum += __shfl_xor(lsum, 16, kWave);
      lsum += __shfl_xor(lsum, 32, kWave);
      float lr[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) lr[r] = __shfl(lsum, 4 * kg + r, kWave);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = cb * 16 + 4 * kg + r;
        int seq, head;
        column(col, ug_o[cb][r], seq, head);
        if (seq < 0) continue;
        if (whole_pair) {
          const float inv = 1.f / lr[r];
          uint32_t packed[VW];
#pragma unroll
          for (int k = 0; k < VW; ++k)
            packed[k] = E::pack(acc[cb][2 * k][r] * inv, acc[cb][2 * k + 1][r] * inv);
          char *o = p.out + (seq * p.out_stride_seq + (int64_t)head * HD + n * VE) * ES;
          if constexpr (VW == 4)
            store16(o, Vec16{{packed[0], packed[1], packed[2 % VW], packed[3 % VW]}});
          else if constexpr (VW == 2)
            *reinterpret_cast<uint2 *>(o) = make_uint2(packed[0], packed[1 % VW]);
          else
            *reinterpret_cast<uint32_t *>(o) = packed[0];
        } else {
          float *o = p.part_acc + (partial * COLS + col) * HD + n * VE;
          if constexpr (VE >= 4) {
#pragma unroll
            for (int k = 0; k < VE / 4; ++k)
              *reinterpret_cast<float4 *>(o + 4 * k) = make_float4(acc[cb][4 * k][r], acc[cb][4 * k + 1][r],
                                                                   acc[cb][4 * k + 2][r], acc[cb][4 * k + 3][r]);
          } else {
            *reinterpret_cast<float2 *>(o) = make_float2(acc[cb][0][r], acc[cb][1][r]);
          }
        }
      }
      if (!whole_pair && kg == 0) {
        int seq, head;
        column(cb * 16 + n, ug_q[cb], seq, head);
        if (seq >= 0) {
          p.part_ml[(partial * COLS + cb * 16 + n) * 2] = m[cb];
          p.part_ml[(partial * COLS + cb * 16 + n) * 2 + 1] = lsum;
        }
      }
      m[cb] = kNegInf;
      l[cb] = 0.f;
#pragma unroll
      for (int e = 0; e < VE; ++e) acc[cb][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    if (left > 0) {
      next_pair(p, rows, c);
      seg_blk0 = 0;
      seg = segment_of(c);
      fetch_q();
    }
  };

  auto consume = [&](Vec16 *kk, VChunk<VW> *vv) {
    // The sequence's last tile may be partly filled (never a shared tile).
    int ctx_here = 0x7fffffff;
    const int tok0 = (c.first + c.blk) * BS;
    if (c.blk == c.nb - 1) {
      // (a scalar load: it waits on the scalar counter only, where a vector load would have to
      // be waited for with everything before it, the prefetched tile included)
      int ctx = ctx_lens[c.tseq];
      ctx = ctx < p.max_ctx ? ctx : p.max_ctx;
      if (tok0 + BS > ctx) {
        ctx_here = ctx;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (tok0 + kg + 4 * r >= ctx) {
#pragma unroll
            for (int k = 0; k < VW; ++k) vv[r].w[k] = 0u;
          }
        }
      }
    }
    // token pairs packed per dim: matrix B of p.v, shared by all column blocks
    Pair32 vb[VE];
#pragma unroll
    for (int k = 0; k < VW; ++k) {
      vb[2 * k] = Pair32{__builtin_amdgcn_perm(vv[1].w[k], vv[0].w[k], 0x05040100u),
                         __builtin_amdgcn_perm(vv[3].w[k], vv[2].w[k], 0x05040100u)};
      vb[2 * k + 1] = Pair32{__builtin_amdgcn_perm(vv[1].w[k], vv[0].w[k], 0x07060302u),
                             __builtin_amdgcn_perm(vv[3].w[k], vv[2].w[k], 0x07060302u)};
    }
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      // ---- scores of column n for tokens kg + 4r ---------------------------------
      f32x4_t s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < NK; ++j) s4 = E::qk(kk[j], qreg[cb][j], s4);
      float s[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[r] = s4[r] * p.scale_log2e;
        if (tok0 + kg + 4 * r >= ctx_here) s[r] = kNegInf;
      }
      // ---- lazy running maximum --------------------------------------------------
      const float smax = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
      if (__any(smax > m[cb] + kLazyMaxSlack)) {  // rare after a segment's first tile
        float mx = smax;
        mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
        mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
        const float m_new = fmaxf(m[cb], mx);
        const float alpha = (m[cb] == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m[cb] - m_new);
        l[cb] *= alpha;
        m[cb] = m_new;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float ar = __shfl(alpha, 4 * kg + r, kWave);
#pragma unroll
          for (int e = 0; e < VE; ++e) acc[cb][e][r] *= ar;
        }
      }
      // ---- probabilities, rounded to the element type, as matrix A of p.v --------
      const float ms = (m[cb] == kNegInf) ? 0.f : m[cb];
      float pr[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pr[r] = __builtin_amdgcn_exp2f(s[r] - ms);
        l[cb] += pr[r];
      }
      const Pair32 pa = {E::pack(pr[0], pr[1]), E::pack(pr[2], pr[3])};
#pragma unroll
      for (int e = 0; e < VE; ++e) acc[cb][e] = E::pv(pa, vb[e], acc[cb][e]);
    }
    ++c.blk;
    --left;
    if (c.blk == c.nb || left == 0) finish_segment();
  };

  auto k_from_lds = [&](const char *base, Vec16 *kk) {
#pragma unroll
    for (int j = 0; j < NK; ++j) kk[j] = *reinterpret_cast<const Vec16 *>(base + kld_off + 64 * j);
  };
  auto k_to_lds = [&](char *base, const Vec16 *kk) {
#pragma unroll
    for (int j = 0; j < NK; ++j) *reinterpret_cast<Vec16 *>(base + kst_off[j]) = kk[j];
  };
  auto consume_fetched = [&](Vec16 *kk, VChunk<VW> *vv) {
    k_to_lds(xpose, kk);
    k_from_lds(xpose, kk);
    consume(kk, vv);
  };

  while (left > 0) {
    const int n_win = left < kWave * SW ? left : kWave * SW;
    uint32_t off_lo[SW], off_hi[SW];
    gather_window<BS, SW, ES>(p, rows, lane, n_win, walk, off_lo, off_hi);

    auto issue = [&](int i, Vec16 *kk, VChunk<VW> *vv) {
      const int64_t tile = window_tile_offset(off_lo, off_hi, i);
      const char *kb = p.k_pool + tile;
      const char *vb = p.v_pool + tile;
#pragma unroll
      for (int j = 0; j < NK; ++j) kk[j] = load16(kb + k_off[j]);
#pragma unroll
      for (int j = 0; j < NT; ++j) vv[j] = load_v<VW>(vb + v_off[j]);
      __builtin_amdgcn_sched_barrier(0);
    };

    // Every issue is unconditional (past the window's end it re-reads the last
    // tile), so the waits on the memory counter stay exact and the loop body
    // exists once.
    Vec16 ka[NK], kb[NK];
    VChunk<VW> va[NT], vb[NT];
    const int last = n_win - 1;
    if (COOP && shared) {
      // All NW waves hold the same share.  Slot w of the ring is written by wave
      // w only, between the two barriers of a round, and read by everyone after
      // the first: K rows as the staging tile holds them, V as lane l wrote it.
      auto put = [&](int slot) {
        char *base = lds_tiles + slot * kSlotBytes;
        k_to_lds(base, ka);
        Vec16 *dst = reinterpret_cast<Vec16 *>(base + 16 * KPITCH) + lane;
#pragma unroll
        for (int j = 0; j < NT * VW / 4; ++j) {
          if constexpr (VW == 4)
            dst[j * kWave] = Vec16{{va[j].w[0], va[j].w[1], va[j].w[2 % VW], va[j].w[3 % VW]}};
          else if constexpr (VW == 2)
            dst[j * kWave] = Vec16{{va[2 * j].w[0], va[2 * j].w[1 % VW], va[2 * j + 1].w[0], va[2 * j + 1].w[1 % VW]}};
          else
            dst[j * kWave] = Vec16{{va[0].w[0], va[1].w[0], va[2].w[0], va[3].w[0]}};
        }
      };
      auto get = [&](int slot) {
        const char *base = lds_tiles + slot * kSlotBytes;
        k_from_lds(base, kb);
        const Vec16 *src = reinterpret_cast<const Vec16 *>(base + 16 * KPITCH) + lane;
#pragma unroll
        for (int j = 0; j < NT * VW / 4; ++j) {
          const Vec16 v = src[j * kWave];
          if constexpr (VW == 4) {
            vb[j] = VChunk<VW>{{v.w[0], v.w[1], v.w[2 % VW], v.w[3 % VW]}};
          } else if constexpr (VW == 2) {
            vb[2 * j] = VChunk<VW>{{v.w[0], v.w[1]}};
            vb[2 * j + 1] = VChunk<VW>{{v.w[2], v.w[3]}};
          } else {
#pragma unroll
            for (int t = 0; t < NT; ++t) vb[t] = VChunk<VW>{{v.w[t]}};
          }
        }
      };
      issue(wave < last ? wave : last, ka, va);
      for (int r0 = 0; r0 < n_win; r0 += NW) {
        put(wave);
        __syncthreads();
        const int mine = r0 + NW + wave;  // this wave's tile of the next round
        issue(mine < last ? mine : last, ka, va);
        const int here = n_win - r0 < NW ? n_win - r0 : NW;
        for (int j = 0; j < here; ++j) {
          get(j);
          consume(kb, vb);
        }
        __syncthreads();
      }
    } else {
      issue(0, ka, va);
      for (int i = 0; i < n_win; i += 2) {
        issue(i + 1 < last ? i + 1 : last, kb, vb);
        consume_fetched(ka, va);
        issue(i + 2 < last ? i + 2 : last, ka, va);
        if (i + 1 < n_win) consume_fetched(kb, vb);
      }
    }
  }
  }  // phase
}

template <class E, int HD, int NW, bool PLAN, bool COOP>
bool launch_variant(DecodeKP &kp, size_t lds_bytes, hipStream_t stream) {
  constexpr int BS = 16;
  auto kernel = paged_decode_mfma_kernel<E, HD, BS, NW, PLAN, COOP>;
  constexpr size_t kLdsGranule = 1024;
  constexpr size_t kMaxLds =
      ((PLAN ? kPlanMaxInts * sizeof(int) : 0) + tiles_lds_bytes(HD, NW, COOP) + kLdsGranule - 1) / kLdsGranule * kLdsGranule;
  static const bool ready = [&] {  // more than 64 KB of dynamic LDS has to be asked for
    return kMaxLds <= 64 * 1024 ||
           hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)kMaxLds) == hipSuccess;
  }();
  if (!ready) return false;
  // Workgroups one CU holds with this much LDS.  The plan's share of LDS grows with the batch, so
  // the request is rounded up to whole KiB and the runtime's answer kept per KiB count, for the
  // whole process: a serving loop whose batch size changes from step to step asks once per size
  // class, and a stream capture on any host thread finds the answers a warm-up on another left.
  lds_bytes = (lds_bytes + kLdsGranule - 1) / kLdsGranule * kLdsGranule;
  static std::atomic<int> per_cu_of[kMaxLds / kLdsGranule + 2];  // 0 = not asked yet
  int per_cu = per_cu_of[lds_bytes / kLdsGranule].load(std::memory_order_relaxed);
  if (per_cu == 0) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, NW * kWave, lds_bytes) != hipSuccess || n < 1) n = 1;
    g_occupancy_queries.fetch_add(1, std::memory_order_relaxed);
    per_cu = n;
    per_cu_of[lds_bytes / kLdsGranule].store(n, std::memory_order_relaxed);
  }
  int wgs = per_cu * device_cu_count();
  // Long rows: one workgroup per CU.  A wave keeps two tiles (16 KiB at head dim 128) in flight,
  // so one 4-wave workgroup per CU already has the bytes in flight that cover HBM's latency at its
  // full rate; a second one adds queueing in the memory system and split-K segments (partials to
  // write and merge, G times larger with G query heads per KV head) and no bandwidth: measured
  // 2-3 % slower for G >= 2 at contexts of 1K-8K tokens (G = 1, whose partials are small, runs
  // the same either way and keeps both workgroups).  With short rows the
  // second workgroup pays: it hides the stalls of the row switches (query load, result write),
  // 7 % on 256 sequences of 64-512 tokens.  Cohorts keep both: their two phases overlap across
  // the workgroups of a CU.
  if (!COOP && kp.cohort_size == 1 && kp.group >= 2 && kp.max_ctx >= kLongRowTokens && wgs > device_cu_count()) {
    wgs = device_cu_count();
    // Rows of several thousand tokens: seven workgroups per eight CUs (still a multiple of 8, so
    // the XCD-major deal holds).  Measured +0.85 % at G = 8, +0.9 % at G = 4, +1.1 % at G = 2 with
    // contexts of 1K-8K tokens (768 to 896 waves all the same, 1 024 slower: the requests of the
    // last CUs only lengthen the queues of a memory system that is already full); with contexts
    // up to 1K it loses 4-6 % (there the launch is short and every CU's share of it counts).
    if (kp.max_ctx >= kVeryLongRowTokens) wgs = (wgs - wgs / 8) & ~7;
  }
  if (wgs * NW > kp.max_waves) wgs = kp.max_waves / NW;
  kp.n_waves = wgs * NW;
  hipLaunchKernelGGL(kernel, dim3(wgs), dim3(NW * kWave), lds_bytes, stream, kp);
  return true;
}

// Plain decode and cohorts one wave covers: 4-wave workgroups, no tile ring.
// Wider cohorts: the workgroup is the unit (2, 4 or 8 waves) and shares tiles
// through LDS.  Batches whose row bookkeeping does not fit LDS scan the rows
// per wave and share tiles through the cache only.
template <class E, int HD>
bool launch_one(DecodeKP &kp, hipStream_t stream) {
  const size_t ints = plan_ints(kp.n_seqs, kp.n_cohorts);
  const int unit = 1 << kp.unit_shift;
  if (ints > (size_t)kPlanMaxInts) {
    return unit > kDecodeWavesPerWorkgroup
               ? launch_variant<E, HD, kMaxCohortWaves, false, false>(
                     kp, tiles_lds_bytes(HD, kMaxCohortWaves, false), stream)
               : launch_variant<E, HD, kDecodeWavesPerWorkgroup, false, false>(
                     kp, tiles_lds_bytes(HD, kDecodeWavesPerWorkgroup, false), stream);
  }
  const size_t plan_bytes = ring_offset_ints(kp.n_seqs, kp.n_cohorts) * sizeof(int);
  switch (unit) {
    case 1:
      return launch_variant<E, HD, kDecodeWavesPerWorkgroup, true, false>(
          kp, plan_bytes + tiles_lds_bytes(HD, kDecodeWavesPerWorkgroup, false), stream);
    case 2: return launch_variant<E, HD, 2, true, true>(kp, plan_bytes + tiles_lds_bytes(HD, 2, true), stream);
    case 4: return launch_variant<E, HD, 4, true, true>(kp, plan_bytes + tiles_lds_bytes(HD, 4, true), stream);
    case 8: return launch_variant<E, HD, 8, true, true>(kp, plan_bytes + tiles_lds_bytes(HD, 8, true), stream);
    default: return false;
  }
}

template <class E>
bool launch_hd(DecodeKP &kp, int hd, hipStream_t stream) {
  switch (hd) {
    case 32: return launch_one<E, 32>(kp, stream);
    case 64: return launch_one<E, 64>(kp, stream);
    case 128: return launch_one<E, 128>(kp, stream);
    default: return false;
  }
}

}  // namespace

long long decode_occupancy_queries() { return g_occupancy_queries.load(std::memory_order_relaxed); }

bool launch_decode_mfma_main(DecodeKP &kp, int dtype, int hd, hipStream_t stream) {
  if (kp.gt < 1 || kp.gt > kCohortColumnsPerWave || (1 << kp.unit_shift) > kMaxCohortWaves) return false;
  switch (dtype) {
    case IC_DTYPE_BF16: return launch_hd<MfmaBf16>(kp, hd, stream);
    case IC_DTYPE_F16: return launch_hd<MfmaF16>(kp, hd, stream);
    default: return false;
  }
}

}  // namespace decode
}  // namespace ic
