// Chunked prefill against the block KV cache: the MFMA path.
//
// Each sequence brings a chunk of C new query tokens whose K/V rows are
// already in the pool; query row r sees keys j <= (L - C) + r (L = context
// length).  This is the reference's dense attention
// (ironcore/layers/attention.py:68-142) with sq = C, sk = L and the causal
// mask of ironcore/language_model.py:109-114 shifted by the cached prefix; with
// causal = 0 every row sees all L keys (the attention_mask=None case).  Query
// head h reads KV head h / G (attention.py:95-102).
//
// A dense contraction, so it runs on the matrix cores
// (v_mfma_f32_32x32x16 bf16/f16, fp32 accumulate), flash-attention style:
//
//  * grid = (query tile of 128 rows, query head, sequence); 4 waves, each
//    owning 32 query rows for the whole K/V sweep.  The wave's Q rows stay in
//    registers as MFMA B operands.
//  * K/V are walked in tiles of 64 tokens (4 pool blocks).  Each thread
//    fetches its 16-byte pieces of the next tile through the block table
//    while the current tile is being used, then parks them in LDS row-major
//    ([token][dim], padded pitch).
//  * Scores are computed TRANSPOSED, S^T = K Q^T: in the MFMA result layout a
//    lane then holds one query column, so the softmax row maximum and row sum
//    are in-lane reductions plus one exchange between the two lane halves,
//    and the rescale of the output accumulator is a per-lane scalar.
//  * O^T += V^T P^T: the probabilities, rounded to the element type, are
//    already in B-operand order (with a fixed permutation of the token index
//    inside each 16-token step), and the matching V^T operand is read from
//    the row-major LDS tile with the transposing LDS read
//    (ds_read_b64_tr_b16), which hands each lane 4 consecutive tokens of one
//    head-dim column.  No transpose pass over V is needed.
//  * Tiles wholly above the causal diagonal are skipped; only tiles that touch
//    it pay for the mask.  Rows past the context length are zero-filled when
//    the tile is staged, so stale pool contents cannot leak.
//
// FLOPs per launch (what utilisation is quoted against): 4*hn*hd per visible
// (query, key) pair = 4*hn*hd * sum_i (C_i*P_i + C_i*(C_i+1)/2).
#include "ic_device.h"
#include "ic_internal.h"
#include "../../include/ironcore_paged.h"

namespace ic {

namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;

struct PrefillKP {
  const char *q;
  const char *k_pool;
  const char *v_pool;
  const int32_t *block_tables;
  const int32_t *context_lens;
  const int32_t *cu_seqlens_q;
  char *out;
  int64_t q_stride_token;    // elements
  int64_t out_stride_token;  // elements
  int64_t stride_block;
  int64_t stride_head;
  int64_t stride_token;
  int64_t bt_stride;
  int64_t num_blocks;
  int block_size;
  int block_shift;  // log2(block_size) when it is a power of two, else -1
  int group;        // query heads per KV head
  int causal;
  float scale_log2e;
};

constexpr float kNegInf = -__builtin_huge_valf();

// MFMA wrappers per element type: operands are 8 packed 16-bit values.
struct MmaBf16 {
  using T = __bf16;
  static __device__ __forceinline__ f32x16_t mma(const Vec16 &a, const Vec16 &b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    bf16x2_t v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};
struct MmaF16 {
  using T = _Float16;
  static __device__ __forceinline__ f32x16_t mma(const Vec16 &a, const Vec16 &b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f16x2_t v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};

constexpr int kPrefillThreads = 256;
constexpr int kBM = 128;  // query rows per workgroup (32 per wave)
constexpr int kBN = 64;   // tokens per K/V tile

template <class M, int HD>
__global__ __launch_bounds__(kPrefillThreads) void paged_prefill_kernel(const PrefillKP p) {
  using T = typename M::T;
  constexpr int KS = HD / 16;          // k-steps of the QK contraction
  constexpr int OB = HD / 32;          // 32-wide blocks of the output head dim
  constexpr int TB = kBN / 32;         // 32-token blocks per tile
  constexpr int CPR = HD / 8;          // 16-byte chunks per token row
  constexpr int NCH = kBN * CPR / kPrefillThreads;  // chunks per thread per tile
  constexpr int KP = HD * 2 + 16;      // K tile pitch in bytes (bank-conflict-free b128 reads)
  constexpr int VP = HD * 2 + 64;      // V tile pitch in bytes (conflict-free transposing reads)
  static_assert(kBN * CPR % kPrefillThreads == 0, "tile staging shape");

  __shared__ __attribute__((aligned(16))) char s_k[kBN * KP];
  __shared__ __attribute__((aligned(16))) char s_v[kBN * VP];

  const int seq = blockIdx.z;
  const int h = blockIdx.y;
  const int q0 = blockIdx.x * kBM;
  const int q_lo = p.cu_seqlens_q[seq];
  int L = p.context_lens[seq];
  int C = p.cu_seqlens_q[seq + 1] - q_lo;
  if (L < 0) L = 0;
  if (C > L) C = L;  // a chunk cannot be longer than its context
  if (q0 >= C) return;
  const int P = L - C;  // cached prefix
  const int kvh = h / p.group;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int n = lane & 31;   // query column of this lane within the wave's 32 rows
  const int hh = lane >> 5;  // which half of each k-step this lane feeds

  const int my_q = q0 + wave * 32 + n;
  const bool q_valid = my_q < C;
  const int64_t q_row = q_lo + (q_valid ? my_q : C - 1);
  // last key this query row may see
  const int limit = p.causal ? P + (q_valid ? my_q : C - 1) : L - 1;

  Vec16 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = load16(p.q + (q_row * p.q_stride_token + (int64_t)h * HD + ks * 16 + hh * 8) * 2);

  f32x16_t o[OB];
#pragma unroll
  for (int ob = 0; ob < OB; ++ob)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[ob][i] = 0.f;
  float m = kNegInf, l = 0.f;

  int kv_end = p.causal ? P + q0 + kBM : L;  // keys any row of this tile can see
  kv_end = kv_end < L ? kv_end : L;
  const int n_tiles = (kv_end + kBN - 1) / kBN;

  // ---- tile staging: global -> registers -> LDS --------------------------------
  Vec16 kst[NCH], vst[NCH];
  auto fetch = [&](int tile) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int chunk = tid + kPrefillThreads * i;
      const int row = chunk / CPR;
      const int cc = chunk - row * CPR;
      const int tok = tile * kBN + row;
      kst[i] = Vec16{{0u, 0u, 0u, 0u}};
      vst[i] = Vec16{{0u, 0u, 0u, 0u}};
      if (tok < L) {
        int blk, off;
        if (p.block_shift >= 0) {
          blk = tok >> p.block_shift;
          off = tok & (p.block_size - 1);
        } else {
          blk = tok / p.block_size;
          off = tok - blk * p.block_size;
        }
        blk = blk < p.bt_stride ? blk : (int)p.bt_stride - 1;
        int64_t phys = p.block_tables[seq * p.bt_stride + blk];
        // A corrupt table entry must not become an out-of-pool address.
        phys = phys < 0 ? 0 : phys;
        phys = phys >= p.num_blocks ? p.num_blocks - 1 : phys;
        const int64_t at =
            (phys * p.stride_block + kvh * p.stride_head + off * p.stride_token + cc * 8) * 2;
        kst[i] = load16(p.k_pool + at);
        vst[i] = load16(p.v_pool + at);
      }
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int chunk = tid + kPrefillThreads * i;
      const int row = chunk / CPR;
      const int cc = chunk - row * CPR;
      store16(s_k + row * KP + cc * 16, kst[i]);
      store16(s_v + row * VP + cc * 16, vst[i]);
    }
  };

  // per-lane LDS offsets
  const int k_lane = n * KP + hh * 16;                                   // + tb*32*KP + ks*32
  const int v_lane = (4 * hh + (lane & 15) / 4) * VP + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

  fetch(0);
  for (int tile = 0; tile < n_tiles; ++tile) {
    park();
    __syncthreads();
    if (tile + 1 < n_tiles) fetch(tile + 1);

    // ---- S^T = K Q^T ------------------------------------------------------------
    f32x16_t s[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[tb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const Vec16 a = load16(s_k + k_lane + tb * 32 * KP + ks * 32);
        s[tb] = M::mma(a, qf[ks], s[tb]);
      }
    }
    // s[tb][i] is (token tile*64 + tb*32 + 4*hh + 8*(i/4) + i%4, query n)
    const int tok_base = tile * kBN + 4 * hh;
    const bool need_mask = p.causal ? (tile * kBN + kBN - 1 > P + q0) : (tile * kBN + kBN > L);
    float mx = kNegInf;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float x = s[tb][i] * p.scale_log2e;
        if (need_mask) {
          const int tok = tok_base + tb * 32 + 8 * (i / 4) + (i & 3);
          x = tok > limit ? kNegInf : x;
        }
        s[tb][i] = x;
        mx = fmaxf(mx, x);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m, mx);
    const float ms = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - ms);
    m = m_new;
    float ps = 0.f;
    Vec16 pb[kBN / 16];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = __builtin_amdgcn_exp2f(s[tb][i] - ms);
        const float p1 = __builtin_amdgcn_exp2f(s[tb][i + 1] - ms);
        ps += p0 + p1;
        pb[2 * tb + i / 8].w[(i & 7) / 2] = M::pack2(p0, p1);
      }
    }
    l = l * alpha + ps;
#pragma unroll
    for (int ob = 0; ob < OB; ++ob)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[ob][i] *= alpha;

    // ---- O^T += V^T P^T -----------------------------------------------------------
#pragma unroll
    for (int ob = 0; ob < OB; ++ob) {
#pragma unroll
      for (int kk = 0; kk < kBN / 16; ++kk) {
        const char *at = s_v + v_lane + kk * 16 * VP + ob * 64;
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t *)(at));
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t *)(at + 8 * VP));
        const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        o[ob] = M::mma(__builtin_bit_cast(Vec16, both), pb[kk], o[ob]);
      }
    }
    __syncthreads();
  }

  // ---- normalise and store -------------------------------------------------------
  l += __shfl_xor(l, 32, kWave);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (q_valid) {
    T *orow = reinterpret_cast<T *>(p.out) + (q_lo + my_q) * p.out_stride_token + (int64_t)h * HD;
#pragma unroll
    for (int ob = 0; ob < OB; ++ob) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = ob * 32 + 4 * hh + 8 * j;
        uint2 w;
        w.x = M::pack2(o[ob][4 * j] * inv, o[ob][4 * j + 1] * inv);
        w.y = M::pack2(o[ob][4 * j + 2] * inv, o[ob][4 * j + 3] * inv);
        *reinterpret_cast<uint2 *>(orow + d) = w;
      }
    }
  }
}

template <class M>
int launch_hd(const PrefillKP &kp, const PrefillArgs &a, hipStream_t stream) {
  const dim3 grid((a.max_chunk_len + kBM - 1) / kBM, a.hn, a.n_seqs);
  switch (a.hd) {
    case 64:
      hipLaunchKernelGGL((paged_prefill_kernel<M, 64>), grid, dim3(kPrefillThreads), 0, stream, kp);
      break;
    case 128:
      hipLaunchKernelGGL((paged_prefill_kernel<M, 128>), grid, dim3(kPrefillThreads), 0, stream, kp);
      break;
    default:
      return IC_ERR_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? IC_OK : IC_ERR_LAUNCH;
}

}  // namespace

int launch_paged_prefill(const PrefillArgs &a, hipStream_t stream) {
  PrefillKP kp;
  kp.q = (const char *)a.q;
  kp.k_pool = (const char *)a.k_pool;
  kp.v_pool = (const char *)a.v_pool;
  kp.block_tables = a.block_tables;
  kp.context_lens = a.context_lens;
  kp.cu_seqlens_q = a.cu_seqlens_q;
  kp.out = (char *)a.out;
  kp.q_stride_token = a.q_stride_token;
  kp.out_stride_token = a.out_stride_token;
  kp.stride_block = a.pool.stride_block;
  kp.stride_head = a.pool.stride_head;
  kp.stride_token = a.pool.stride_token;
  kp.bt_stride = a.block_table_stride;
  kp.num_blocks = a.pool.num_blocks;
  kp.block_size = a.pool.block_size;
  kp.block_shift = -1;
  for (int s = 0; s < 31; ++s)
    if ((1 << s) == a.pool.block_size) kp.block_shift = s;
  kp.group = a.hn / a.gn;
  kp.causal = a.causal;
  kp.scale_log2e = a.scale * 1.4426950408889634f;
  if ((int64_t)a.max_chunk_len + kBM - 1 >= (int64_t)65535 * kBM || a.hn > 65535 || a.n_seqs > 65535)
    return IC_ERR_UNSUPPORTED;
  switch (a.dtype) {
    case IC_DTYPE_BF16: return launch_hd<MmaBf16>(kp, a, stream);
    case IC_DTYPE_F16: return launch_hd<MmaF16>(kp, a, stream);
    default: return IC_ERR_UNSUPPORTED;  // fp32 has no MFMA path here
  }
}

}  // namespace ic
