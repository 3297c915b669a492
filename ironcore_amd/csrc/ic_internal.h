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

// KV append with rotary embedding: the plain append's arguments (k_new / v_new
// may be null: rotate the query rows only) plus the query rows and the tables.
struct RopeAppendArgs {
  AppendArgs append;
  void *q;                 // [n_tokens, hn, hd] rotated in place, or nullptr
  int64_t q_stride_token;  // elements
  int hn;
  const int32_t *positions;  // [n_tokens] row of the tables each token uses
  const float *cos_table;    // [table_rows, hd / 2]
  const float *sin_table;
  int64_t table_rows;
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
  int min_chunk_tokens;  // smallest split-K share (multiple of block_size)
  int32_t *cum_blocks;   // workspace: [n_seqs + 1], then [n_cohorts + 1] with cohorts
  int64_t shared_slot0;  // first partial slot of the shared phase
  float *part_ml;        // workspace: [partial slots, 2]
  float *part_acc;       // workspace: [partial slots, hd]
  int cohort_size;       // 1 = no shared prefixes
  const int32_t *cohort_shared_blocks;  // [ceil(n_seqs / cohort_size)], or nullptr
  int max_waves;         // the workspace holds partials for this many waves (0 = kMaxDecodeWaves)
  int dtype;
  // optional key mask (fp32 kernel only): byte (sequence, query head, key) at
  // seq*key_mask_stride_seq + head*key_mask_stride_head + key, nonzero = visible
  const uint8_t *key_mask = nullptr;
  int64_t key_mask_stride_seq = 0;
  int64_t key_mask_stride_head = 0;
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
  // optional byte mask (nullptr = the causal rule / no mask): element (sequence, head, chunk row,
  // key) at seq*mask_stride_seq + head*mask_stride_head + row*mask_stride_row + key
  const uint8_t *mask = nullptr;
  int64_t mask_stride_seq = 0;
  int64_t mask_stride_head = 0;
  int64_t mask_stride_row = 0;
  int64_t mask_keys = 0;  // keys a mask row covers; keys from there on are hidden
};

// Each returns IC_OK, IC_ERR_UNSUPPORTED (no kernel built for this
// dtype/shape) or IC_ERR_LAUNCH.
int launch_kv_append(const AppendArgs &a, hipStream_t stream);
int launch_rope_kv_append(const RopeAppendArgs &a, hipStream_t stream);
int launch_paged_decode(const DecodeArgs &a, hipStream_t stream);
int launch_paged_prefill(const PrefillArgs &a, hipStream_t stream);

constexpr int kDefaultMinChunkTokens = 16;  // one tile: short batches spread over all waves
// Upper bound on the waves of one decode launch (sizes the workspace): 8 waves
// on each of the 4 SIMDs of up to 512 CUs.
constexpr int kMaxDecodeWaves = 16384;

inline int elem_size(int dtype) { return dtype == 2 ? 4 : 2; }

// Query heads one wave carries for a KV head with `group` query heads; larger
// groups are cut into ceil(group / 8) sub-groups.
inline int decode_heads_per_wave(int group) { return group <= 8 ? group : 8; }

// Shared-prefix cohorts: a wave carries 16 matrix columns, i.e. the heads of
// 16 / group members; up to 8 waves of one workgroup walk a cohort's shared
// tiles together, each with its own members.
constexpr int kCohortColumnsPerWave = 16;
constexpr int kMaxCohortWaves = 8;

// Work layout of one decode call.
struct DecodeLayout {
  int cols;        // matrix columns per partial slot
  int nsub;        // query sub-groups per KV head
  int n_cohorts;   // 0 without cohorts
  int spw;         // cohort members per wave in the shared phase
  int unit_shift;  // log2 of the waves that share one cohort's tiles
  bool ok;         // false: the cohort does not fit (group > 16 or too many members)
};
inline DecodeLayout decode_layout(int n_seqs, int hn, int gn, int cohort_size) {
  const int group = hn / gn;
  if (cohort_size <= 1) {
    const int gt = decode_heads_per_wave(group);
    return {gt, (group + gt - 1) / gt, 0, 1, 0, true};
  }
  if (group > kCohortColumnsPerWave) return {0, 0, 0, 0, 0, false};
  int spw = kCohortColumnsPerWave / group;
  if (spw > cohort_size) spw = cohort_size;
  const int waves = (cohort_size + spw - 1) / spw;
  int shift = 0;
  while ((1 << shift) < waves) ++shift;
  if ((1 << shift) > kMaxCohortWaves) return {0, 0, 0, 0, 0, false};
  return {spw * group, 1, (n_seqs + cohort_size - 1) / cohort_size, spw, shift, true};
}

// Split-K workspace layout for the decode entry points.
struct DecodeWorkspace {
  size_t cum_bytes;     // int32 [n_seqs + 1] then [n_cohorts + 1], padded to 256
  size_t ml_bytes;      // float [slots, 2], padded to 256
  size_t acc_bytes;     // float [slots, hd]
  size_t shared_slot0;  // first partial slot of the shared phase
  size_t total() const { return cum_bytes + ml_bytes + acc_bytes; }
};
inline DecodeWorkspace decode_workspace(int n_seqs, int hn, int gn, int hd, int cohort_size,
                                        int max_waves = kMaxDecodeWaves) {
  const DecodeLayout lay = decode_layout(n_seqs, hn, gn, cohort_size);
  const size_t pairs = (size_t)gn * lay.nsub;
  // one partial per (wave, row, pair) segment: fewer than waves + rows*pairs of them; the shared
  // phase has one per (unit, cohort, pair) segment and wave of the unit
  const size_t own = (size_t)max_waves + (size_t)n_seqs * pairs;
  const size_t shared = lay.n_cohorts > 0
                            ? (size_t)max_waves + (((size_t)lay.n_cohorts * pairs) << lay.unit_shift)
                            : 0;
  const size_t slots = (own + shared) * lay.cols;
  auto pad = [](size_t n) { return (n + 255) & ~(size_t)255; };
  return {pad(((size_t)n_seqs + 1 + (size_t)lay.n_cohorts + 1) * sizeof(int32_t)),
          pad(slots * 2 * sizeof(float)), slots * hd * sizeof(float), own};
}

// Compute units of the current device (cached per device ordinal).
int device_cu_count();

// Launches the matrix-rate probe (mfma_probe.hip); returns the launch's flop count or a negative IC_ERR_*.
int64_t launch_mfma_probe(int iters, void *sink, hipStream_t stream);

}  // namespace ic
