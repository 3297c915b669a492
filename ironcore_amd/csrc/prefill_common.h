// Pieces shared by the chunked-prefill kernels (the 16-bit matrix-core kernel
// of paged_prefill.hip and the fp32 one of paged_prefill_f32.hip): kernel
// parameters, the values that stand for hidden scores, the exchange between a
// wave's two lane halves.
#pragma once

#include "ic_device.h"
#include "ic_internal.h"

namespace ic {
namespace prefill {

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
  int block_size;   // a multiple of 16 tokens
  int block_shift;  // log2(block_size) when it is a power of two, else -1
  uint32_t block_magic;  // row / block_size == mulhi(row, block_magic): 2^32 / block_size for a power of two
                         // (exact for every row), else floor(2^32 / block_size) + 1 (exact below 2^32 / block_size)
  int group;        // query heads per KV head
  int gn;           // KV heads
  int n_units;      // n_seqs * gn
  int n_qtiles;     // query tiles per chunk (grid sizing)
  int causal;
  float scale_log2e;
  // General attention mask (MASK variant): byte (sequence i, head h, chunk row r, key j) at
  // mask[i*mask_stride_seq + h*mask_stride_head + r*mask_stride_row + j], nonzero = visible.
  const uint8_t *mask;
  int64_t mask_stride_seq;
  int64_t mask_stride_head;
  int64_t mask_stride_row;
  int mask_keys;  // keys a mask row covers: keys from there on are hidden and never read
};

constexpr float kNegInf = -__builtin_huge_valf();
// Raw score of a key the mask hides.  The reference fills hidden scores with the FINITE minimum
// of the element type (attention.py:66,115-117), not -inf: beside any visible key the hidden ones
// get probability 0 either way, but a row with no visible key at all becomes a uniform average of
// V over the whole context.  A power of two, so that its product with the scale is exact and the
// exponent of a fully hidden row is exactly 0.
constexpr float kHiddenScore = -0x1p100f;

// x of this lane and x of lane ^ 32, as a pair (v_permlane32_swap: a vector-ALU
// exchange, where a shuffle would be an LDS operation and share its counter).
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void both_halves(float x, float &a, float &b) {
  const unsigned int u = __builtin_bit_cast(unsigned int, x);
  const u32x2_t r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  unsigned int r0 = r[0], r1 = r[1];
  // Opaque to the optimiser, which otherwise takes the two results of the swap
  // for the same value and folds max(r0, r1) to r0.
  asm("" : "+v"(r0), "+v"(r1));
  a = __builtin_bit_cast(float, r0);
  b = __builtin_bit_cast(float, r1);
}

constexpr float kLazySlack = 8.0f;  // log2 units

// fp32 pools: the kernel of paged_prefill_f32.hip (same parameters, same grid rules of its own).
int launch_paged_prefill_f32(PrefillKP kp, const PrefillArgs &a, hipStream_t stream);

}  // namespace prefill
}  // namespace ic
