// Host-side launch interfaces between the C ABI (ic_api.hip) and the kernel
// translation units.  Arguments have been validated by the caller.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace ic {

struct PoolLayout {
  int64_t stride_block;  // elements
  int64_t stride_head;
  int64_t stride_token;
  int64_t num_blocks;
  int block_size;
};

struct AppendArgs {
  const void *k_new;
  const void *v_new;
  int64_t new_stride_token;
  void *k_pool;
  void *v_pool;
  PoolLayout pool;
  const int64_t *slot_mapping;
  int64_t n_tokens;
  int gn;
  int hd;
  int dtype;
};

struct DecodeArgs {
  void *out;
  int64_t out_stride_seq;
  const void *q;
  int64_t q_stride_seq;
  const void *k_pool;
  const void *v_pool;
  PoolLayout pool;
  const int32_t *block_tables;
  int64_t block_table_stride;
  const int32_t *context_lens;
  int n_seqs;
  int hn;
  int gn;
  int hd;
  int max_context_len;
  float scale;
  int part_tokens;
  int n_parts;     // ceil(max_context_len / part_tokens)
  float *part_ml;  // [n_seqs, hn, n_parts, 2]
  float *part_acc; // [n_seqs, hn, n_parts, hd]
  int dtype;
};

struct PrefillArgs {
  void *out;
  int64_t out_stride_token;
  const void *q;
  int64_t q_stride_token;
  const void *k_pool;
  const void *v_pool;
  PoolLayout pool;
  const int32_t *block_tables;
  int64_t block_table_stride;
  const int32_t *context_lens;
  const int32_t *cu_seqlens_q;
  int n_seqs;
  int max_chunk_len;
  int hn;
  int gn;
  int hd;
  float scale;
  int causal;
  int dtype;
};

// Each returns IC_OK, IC_ERR_UNSUPPORTED (no kernel built for this
// dtype/shape) or IC_ERR_LAUNCH.
int launch_kv_append(const AppendArgs &a, hipStream_t stream);
int launch_paged_decode(const DecodeArgs &a, hipStream_t stream);
int launch_paged_prefill(const PrefillArgs &a, hipStream_t stream);

constexpr int kDefaultPartTokens = 256;
constexpr int kMaxPartBlocks = 64;  // blocks per split-K partition: one block-table entry per lane

inline int elem_size(int dtype) { return dtype == 2 ? 4 : 2; }

}  // namespace ic
