// Rotary position embedding fused into the KV append.
//
// A transformer layer with rotary embeddings rotates its query and key rows
// right after the projections and before attention
// (reference: ironcore/models/transformer.py:95-98 calling
// ironcore/layers/positional_embedding/rotary.py:53-83).  With a block KV
// cache that is also the moment the new K/V rows enter the pool, so one pass
// does all three: rotate Q in place, rotate K into its pool slots, copy V into
// its pool slots.  Rotated keys are stored, so a cached key is never rotated
// again.
//
// Arithmetic is the reference's (rotary.py:69-83), element pairs (2i, 2i+1):
//     out[2i]   = x[2i] * cos - x[2i+1] * sin
//     out[2i+1] = x[2i] * sin + x[2i+1] * cos
// in fp32 with every product and sum rounded on its own (no fused
// multiply-add), then rounded to the element type: bit-identical to the same
// expression evaluated by torch on the CPU.  cos/sin come from the caller's
// fp32 tables [rows, hd/2] (the reference caches exactly such tables,
// rotary.py:36-51), indexed by positions[token]: WHICH row a token uses is the
// caller's decision (its true position in the sequence for a cached decoder).
//
// HBM-bound: one lane handles one 16-byte chunk (4 pairs in 16-bit types, 2
// in fp32) and the matching 16 or 8 bytes of each table row; blockIdx.z picks
// K, V or Q.  Algorithmic traffic: K and V rows read once and written once,
// Q rows read and written in place, 12 bytes of slot and position per token;
// the table rows in use stay in cache.
#include "ic_device.h"
#include "ic_internal.h"
#include "../../include/ironcore_paged.h"

namespace ic {

namespace {

constexpr int kRopeThreads = 256;

struct RopeKP {
  char *q;                // rotated in place, or nullptr
  const char *k_new;      // or nullptr: no K/V work
  const char *v_new;
  char *k_pool;
  char *v_pool;
  const int64_t *slot_mapping;
  const int32_t *positions;
  const float *cos_table;
  const float *sin_table;
  int64_t q_stride_bytes;
  int64_t new_stride_bytes;
  int64_t stride_block_bytes;
  int64_t stride_head_bytes;
  int64_t stride_token_bytes;
  int64_t num_slots;
  int64_t table_rows;
  int chunks_per_head;
  int q_chunks;   // per token
  int kv_chunks;  // per token
  int block_size;
  int half_hd;
};

// Products and sums rounded one by one, as a sequence of separate torch ops
// is.  Contraction is off for these operations: by default the compiler may
// fuse a product into the following sum (one rounding instead of two), and
// for fp16 inputs also the widening and the final narrowing.
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c, float s, float &o1, float &o2) {
#pragma clang fp contract(off)
  const float a = x1 * c;
  const float b = x2 * s;
  const float d = x1 * s;
  const float e = x2 * c;
  o1 = a - b;
  o2 = d + e;
}

template <class E>
__device__ __forceinline__ Vec16 rotate_chunk(const Vec16 &x, const float *cs, const float *sn);

template <>
__device__ __forceinline__ Vec16 rotate_chunk<F32>(const Vec16 &x, const float *cs, const float *sn) {
  const float2 c = *reinterpret_cast<const float2 *>(cs);
  const float2 s = *reinterpret_cast<const float2 *>(sn);
  float o[4];
  rotate_pair(__builtin_bit_cast(float, x.w[0]), __builtin_bit_cast(float, x.w[1]), c.x, s.x, o[0], o[1]);
  rotate_pair(__builtin_bit_cast(float, x.w[2]), __builtin_bit_cast(float, x.w[3]), c.y, s.y, o[2], o[3]);
  Vec16 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r.w[i] = __builtin_bit_cast(uint32_t, o[i]);
  return r;
}

template <class E>
__device__ __forceinline__ Vec16 rotate_chunk16(const Vec16 &x, const float *cs, const float *sn) {
  using T = typename E::type;
  const float4 c = *reinterpret_cast<const float4 *>(cs);
  const float4 s = *reinterpret_cast<const float4 *>(sn);
  const float cc[4] = {c.x, c.y, c.z, c.w};
  const float ss[4] = {s.x, s.y, s.z, s.w};
  float f[8];
  E::widen(x, f);
  Vec16 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float o1, o2;
    rotate_pair(f[2 * i], f[2 * i + 1], cc[i], ss[i], o1, o2);
    const T lo = E::narrow(o1), hi = E::narrow(o2);
    r.w[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
  }
  return r;
}
template <>
__device__ __forceinline__ Vec16 rotate_chunk<Bf16>(const Vec16 &x, const float *cs, const float *sn) {
  return rotate_chunk16<Bf16>(x, cs, sn);
}
template <>
__device__ __forceinline__ Vec16 rotate_chunk<F16>(const Vec16 &x, const float *cs, const float *sn) {
  return rotate_chunk16<F16>(x, cs, sn);
}

template <class E>
__global__ __launch_bounds__(kRopeThreads) void rope_kv_append_kernel(const RopeKP p, int64_t t0) {
  constexpr int PAIRS = E::EPL / 2;  // pairs in one 16-byte chunk
  const int64_t t = t0 + blockIdx.y;
  const int part = blockIdx.z;  // 0: K, 1: V, 2: Q
  const int c = blockIdx.x * kRopeThreads + threadIdx.x;
  int64_t pos = p.positions[t];
  pos = pos < 0 ? 0 : pos;
  pos = pos >= p.table_rows ? p.table_rows - 1 : pos;
  if (part == 2) {
    if (p.q == nullptr || c >= p.q_chunks) return;
    const int within = c % p.chunks_per_head;
    char *at = p.q + t * p.q_stride_bytes + (int64_t)c * 16;
    const int64_t trig = pos * p.half_hd + within * PAIRS;
    store16(at, rotate_chunk<E>(load16(at), p.cos_table + trig, p.sin_table + trig));
    return;
  }
  if (p.k_new == nullptr || c >= p.kv_chunks) return;
  const int64_t slot = p.slot_mapping[t];
  if (slot < 0 || slot >= p.num_slots) return;
  const int64_t blk = slot / p.block_size;
  const int64_t off = slot - blk * p.block_size;
  const int head = c / p.chunks_per_head;
  const int within = c - head * p.chunks_per_head;
  const int64_t dst = blk * p.stride_block_bytes + head * p.stride_head_bytes + off * p.stride_token_bytes +
                      (int64_t)within * 16;
  const int64_t src = t * p.new_stride_bytes + (int64_t)c * 16;
  if (part == 1) {
    store16(p.v_pool + dst, load16(p.v_new + src));
  } else {
    const int64_t trig = pos * p.half_hd + within * PAIRS;
    store16(p.k_pool + dst, rotate_chunk<E>(load16(p.k_new + src), p.cos_table + trig, p.sin_table + trig));
  }
}

template <class E>
int launch_typed(const RopeKP &kp, int64_t n_tokens, hipStream_t stream) {
  const int widest = kp.q_chunks > kp.kv_chunks ? kp.q_chunks : kp.kv_chunks;
  dim3 grid((widest + kRopeThreads - 1) / kRopeThreads, 1, 3);
  const int64_t kMaxY = 65535;  // gridDim.y limit: walk longer batches in slices
  for (int64_t t0 = 0; t0 < n_tokens; t0 += kMaxY) {
    grid.y = (unsigned)((n_tokens - t0 < kMaxY) ? n_tokens - t0 : kMaxY);
    hipLaunchKernelGGL(rope_kv_append_kernel<E>, grid, dim3(kRopeThreads), 0, stream, kp, t0);
  }
  return hipGetLastError() == hipSuccess ? IC_OK : IC_ERR_LAUNCH;
}

}  // namespace

int launch_rope_kv_append(const RopeAppendArgs &a, hipStream_t stream) {
  if (a.append.n_tokens == 0) return IC_OK;
  const AppendArgs &ap = a.append;
  const int es = elem_size(ap.dtype);
  RopeKP kp;
  kp.q = (char *)a.q;
  kp.k_new = (const char *)ap.k_new;
  kp.v_new = (const char *)ap.v_new;
  kp.k_pool = (char *)ap.k_pool;
  kp.v_pool = (char *)ap.v_pool;
  kp.slot_mapping = ap.slot_mapping;
  kp.positions = a.positions;
  kp.cos_table = a.cos_table;
  kp.sin_table = a.sin_table;
  kp.q_stride_bytes = a.q_stride_token * es;
  kp.new_stride_bytes = ap.new_stride_token * es;
  kp.stride_block_bytes = ap.pool.stride_block * es;
  kp.stride_head_bytes = ap.pool.stride_head * es;
  kp.stride_token_bytes = ap.pool.stride_token * es;
  kp.num_slots = ap.pool.num_blocks * ap.pool.block_size;
  kp.table_rows = a.table_rows;
  kp.chunks_per_head = ap.hd * es / 16;
  kp.q_chunks = a.q ? kp.chunks_per_head * a.hn : 0;
  kp.kv_chunks = ap.k_new ? kp.chunks_per_head * ap.gn : 0;
  kp.block_size = ap.pool.block_size;
  kp.half_hd = ap.hd / 2;
  switch (ap.dtype) {
    case IC_DTYPE_BF16: return launch_typed<Bf16>(kp, ap.n_tokens, stream);
    case IC_DTYPE_F16: return launch_typed<F16>(kp, ap.n_tokens, stream);
    case IC_DTYPE_F32: return launch_typed<F32>(kp, ap.n_tokens, stream);
    default: return IC_ERR_UNSUPPORTED;
  }
}

}  // namespace ic
