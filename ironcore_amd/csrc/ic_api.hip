// C ABI: argument validation on the host, then dispatch to the kernel
// launchers.  Nothing here allocates, synchronises or keeps state.
#include <atomic>

#include "ic_internal.h"
#include "../../include/ironcore_paged.h"

namespace ic {
namespace decode {
long long decode_occupancy_queries();  // paged_decode_mfma.hip
}
}  // namespace ic

// Device memory of the entry point that may not allocate (ic_paged_decode_static): the decode
// workspace (row prefix sums and split-K partials) lives in this array instead of a buffer the
// caller brings.  Every GPU the library runs on holds its own copy at its own address until the
// process ends; host code reaches it only through the address hipGetSymbolAddress returns for the
// current device (static_scratch below), never through the array's name.
static __device__ __align__(256) unsigned char scratch[IC_STATIC_SCRATCH_BYTES];

namespace {

// Grid cap of the static entry point: 8 waves on each of up to 512 CUs (an MI355X launch uses
// 2048).  It bounds the partial slots, so that the BASELINE decode shapes fit the scratch array.
constexpr int kStaticMaxWaves = 4096;
constexpr int kMaxDevices = 64;

// Address of `scratch` on the current device, looked up once per device; nullptr on failure.
void *static_scratch() {
  static std::atomic<void *> addr[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void *p = addr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    addr[dev].store(p, std::memory_order_release);
  }
  return p;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
bool dtype_ok(int dtype) { return dtype == IC_DTYPE_BF16 || dtype == IC_DTYPE_F16 || dtype == IC_DTYPE_F32; }

// A stride (elements) keeps 16-byte chunks aligned when stride*elem % 16 == 0.
bool stride16(int64_t stride, int es) { return ((stride * es) & 15) == 0; }

int check_pool(int64_t sb, int64_t sh, int64_t st, int gn, int hd, int block_size, int64_t num_blocks,
               int es) {
  if (gn <= 0 || hd <= 0 || block_size <= 0 || num_blocks <= 0) return IC_ERR_BAD_SHAPE;
  if (sb <= 0 || sh <= 0 || st < hd) return IC_ERR_BAD_SHAPE;
  if ((hd * es) % 16 != 0) return IC_ERR_UNSUPPORTED;
  if (!stride16(sb, es) || !stride16(sh, es) || !stride16(st, es)) return IC_ERR_ALIGNMENT;
  return IC_OK;
}

int resolve_min_chunk(int min_chunk_tokens) {
  if (min_chunk_tokens == 0) min_chunk_tokens = ic::kDefaultMinChunkTokens;
  if (min_chunk_tokens < 16 || min_chunk_tokens % 16 != 0) return -1;
  return min_chunk_tokens;
}

// Both decode entry points and the variant on the library's own scratch: checks, then the launch.
// The workspace has partial slots for a grid of at most `max_waves` waves.
int decode_checked(void *out, int64_t out_stride_seq, const void *q, int64_t q_stride_seq,
                   const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                   int64_t pool_stride_head, int64_t pool_stride_token, const int32_t *block_tables,
                   int64_t block_table_stride, const int32_t *context_lens, int n_seqs, int hn, int gn,
                   int hd, int block_size, int64_t num_blocks, int max_context_len, float scale,
                   int min_chunk_tokens, int cohort_size, const int32_t *cohort_shared_blocks,
                   void *workspace, size_t workspace_bytes, int max_waves, int dtype, void *stream,
                   const uint8_t *key_mask = nullptr, int64_t key_mask_stride_seq = 0,
                   int64_t key_mask_stride_head = 0) {
  if (n_seqs < 0 || hn <= 0 || gn <= 0 || hn % gn != 0 || max_context_len < 0 || cohort_size < 1)
    return IC_ERR_BAD_SHAPE;
  if (key_mask != nullptr) {
    if (dtype != IC_DTYPE_F32 || cohort_size != 1) return IC_ERR_UNSUPPORTED;
    if (key_mask_stride_seq < max_context_len || key_mask_stride_head < 0) return IC_ERR_BAD_SHAPE;
  }
  if (!dtype_ok(dtype)) return IC_ERR_UNSUPPORTED;
  const int es = ic::elem_size(dtype);
  if (int rc = check_pool(pool_stride_block, pool_stride_head, pool_stride_token, gn, hd, block_size,
                          num_blocks, es))
    return rc;
  if (n_seqs == 0) return IC_OK;
  if (!out || !q || !k_pool || !v_pool || !block_tables || !context_lens) return IC_ERR_NULL_POINTER;
  if (cohort_size > 1) {
    if (!cohort_shared_blocks) return IC_ERR_NULL_POINTER;
    if (dtype == IC_DTYPE_F32 || !ic::decode_layout(n_seqs, hn, gn, cohort_size).ok) return IC_ERR_UNSUPPORTED;
  }
  if (out_stride_seq < (int64_t)hn * hd || q_stride_seq < (int64_t)hn * hd) return IC_ERR_BAD_SHAPE;
  if (max_context_len == 0) max_context_len = 1;  // all-empty batch: the reduce pass writes zeros
  const int mc = resolve_min_chunk(min_chunk_tokens);
  if (mc < 0) return IC_ERR_BAD_SHAPE;
  const int64_t need_blocks = ((int64_t)max_context_len + block_size - 1) / block_size;
  if (block_table_stride < need_blocks) return IC_ERR_BAD_SHAPE;
  if (!aligned16(q) || !aligned16(k_pool) || !aligned16(v_pool) || !stride16(q_stride_seq, es))
    return IC_ERR_ALIGNMENT;
  // the matrix-core kernel stores 8- or 16-byte pieces of output rows
  if (es == 2 && (!aligned16(out) || !stride16(out_stride_seq, es))) return IC_ERR_ALIGNMENT;
  const ic::DecodeWorkspace ws = ic::decode_workspace(n_seqs, hn, gn, hd, cohort_size, max_waves);
  if (!workspace || workspace_bytes < ws.total() || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return IC_ERR_WORKSPACE;

  ic::DecodeArgs a;
  a.out = out;
  a.out_stride_seq = out_stride_seq;
  a.q = q;
  a.q_stride_seq = q_stride_seq;
  a.k_pool = k_pool;
  a.v_pool = v_pool;
  a.pool = {pool_stride_block, pool_stride_head, pool_stride_token, num_blocks, block_size};
  a.block_tables = block_tables;
  a.block_table_stride = block_table_stride;
  a.context_lens = context_lens;
  a.n_seqs = n_seqs;
  a.hn = hn;
  a.gn = gn;
  a.hd = hd;
  a.max_context_len = max_context_len;
  a.scale = scale;
  a.min_chunk_tokens = mc;
  char *wsp = static_cast<char *>(workspace);
  a.cum_blocks = reinterpret_cast<int32_t *>(wsp);
  a.part_ml = reinterpret_cast<float *>(wsp + ws.cum_bytes);
  a.part_acc = reinterpret_cast<float *>(wsp + ws.cum_bytes + ws.ml_bytes);
  a.shared_slot0 = (int64_t)ws.shared_slot0;
  a.cohort_size = cohort_size;
  a.cohort_shared_blocks = cohort_shared_blocks;
  a.max_waves = max_waves;
  a.key_mask = key_mask;
  a.key_mask_stride_seq = key_mask_stride_seq;
  a.key_mask_stride_head = key_mask_stride_head;
  a.dtype = dtype;
  return ic::launch_paged_decode(a, static_cast<hipStream_t>(stream));
}

int prefill_checked(void *out, int64_t out_stride_token, const void *q, int64_t q_stride_token,
                    const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                    int64_t pool_stride_head, int64_t pool_stride_token, const int32_t *block_tables,
                    int64_t block_table_stride, const int32_t *context_lens, const int32_t *cu_seqlens_q,
                    int n_seqs, int max_chunk_len, int hn, int gn, int hd, int block_size,
                    int64_t num_blocks, float scale, int causal, const uint8_t *mask,
                    int64_t mask_stride_seq, int64_t mask_stride_head, int64_t mask_stride_row,
                    int64_t mask_keys, int dtype, void *stream) {
  if (n_seqs < 0 || max_chunk_len < 0 || hn <= 0 || gn <= 0 || hn % gn != 0) return IC_ERR_BAD_SHAPE;
  if (!dtype_ok(dtype)) return IC_ERR_UNSUPPORTED;
  const int es = ic::elem_size(dtype);
  if (int rc = check_pool(pool_stride_block, pool_stride_head, pool_stride_token, gn, hd, block_size,
                          num_blocks, es))
    return rc;
  if (n_seqs == 0 || max_chunk_len == 0) return IC_OK;
  if (!out || !q || !k_pool || !v_pool || !block_tables || !context_lens || !cu_seqlens_q)
    return IC_ERR_NULL_POINTER;
  if (out_stride_token < (int64_t)hn * hd || q_stride_token < (int64_t)hn * hd) return IC_ERR_BAD_SHAPE;
  if (block_table_stride <= 0) return IC_ERR_BAD_SHAPE;
  if (!aligned16(q) || !aligned16(out) || !aligned16(k_pool) || !aligned16(v_pool) ||
      !stride16(q_stride_token, es) || !stride16(out_stride_token, es))
    return IC_ERR_ALIGNMENT;
  ic::PrefillArgs a;
  a.out = out;
  a.out_stride_token = out_stride_token;
  a.q = q;
  a.q_stride_token = q_stride_token;
  a.k_pool = k_pool;
  a.v_pool = v_pool;
  a.pool = {pool_stride_block, pool_stride_head, pool_stride_token, num_blocks, block_size};
  a.block_tables = block_tables;
  a.block_table_stride = block_table_stride;
  a.context_lens = context_lens;
  a.cu_seqlens_q = cu_seqlens_q;
  a.n_seqs = n_seqs;
  a.max_chunk_len = max_chunk_len;
  a.hn = hn;
  a.gn = gn;
  a.hd = hd;
  a.scale = scale;
  a.causal = causal;
  a.dtype = dtype;
  a.mask = mask;
  a.mask_stride_seq = mask_stride_seq;
  a.mask_stride_head = mask_stride_head;
  a.mask_stride_row = mask_stride_row;
  a.mask_keys = mask_keys;
  return ic::launch_paged_prefill(a, static_cast<hipStream_t>(stream));
}

}  // namespace

namespace ic {

int device_cu_count() {
  static std::atomic<int> cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  int n = cache[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1)
      n = 256;
    cache[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

}  // namespace ic

extern "C" {

int ic_version(void) { return 200; }

int64_t ic_decode_occupancy_queries(void) { return ic::decode::decode_occupancy_queries(); }

int64_t ic_mfma_probe(int iters, void *sink, void *stream) {
  if (sink == nullptr) return IC_ERR_NULL_POINTER;
  if (iters < 1 || iters > (1 << 24)) return IC_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(sink) & 3) != 0) return IC_ERR_ALIGNMENT;
  return ic::launch_mfma_probe(iters, sink, static_cast<hipStream_t>(stream));
}

const char *ic_error_string(int code) {
  switch (code) {
    case IC_OK: return "ok";
    case IC_ERR_NULL_POINTER: return "a required pointer is NULL";
    case IC_ERR_BAD_SHAPE: return "a size or stride is non-positive or inconsistent";
    case IC_ERR_UNSUPPORTED: return "no kernel built for this dtype / head_dim / group / block size";
    case IC_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case IC_ERR_LAUNCH: return "kernel launch failed";
    case IC_ERR_ALIGNMENT: return "pointer or stride is not 16-byte aligned";
    case IC_ERR_STATIC_LIMIT:
      return "the batch needs more scratch than the library's static buffer holds (IC_STATIC_SCRATCH_BYTES); "
             "use ic_paged_decode with a caller-provided workspace";
    default: return "unknown error code";
  }
}

int ic_kv_append(const void *k_new, const void *v_new, int64_t new_stride_token, void *k_pool,
                 void *v_pool, int64_t pool_stride_block, int64_t pool_stride_head,
                 int64_t pool_stride_token, const int64_t *slot_mapping, int64_t n_tokens, int gn,
                 int hd, int block_size, int64_t num_blocks, int dtype, void *stream) {
  if (n_tokens < 0) return IC_ERR_BAD_SHAPE;
  if (!dtype_ok(dtype)) return IC_ERR_UNSUPPORTED;
  const int es = ic::elem_size(dtype);
  if (int rc = check_pool(pool_stride_block, pool_stride_head, pool_stride_token, gn, hd, block_size,
                          num_blocks, es))
    return rc;
  if (n_tokens == 0) return IC_OK;
  if (!k_new || !v_new || !k_pool || !v_pool || !slot_mapping) return IC_ERR_NULL_POINTER;
  if (new_stride_token < (int64_t)gn * hd) return IC_ERR_BAD_SHAPE;
  if (!aligned16(k_new) || !aligned16(v_new) || !aligned16(k_pool) || !aligned16(v_pool) ||
      !stride16(new_stride_token, es))
    return IC_ERR_ALIGNMENT;
  ic::AppendArgs a;
  a.k_new = k_new;
  a.v_new = v_new;
  a.new_stride_token = new_stride_token;
  a.k_pool = k_pool;
  a.v_pool = v_pool;
  a.pool = {pool_stride_block, pool_stride_head, pool_stride_token, num_blocks, block_size};
  a.slot_mapping = slot_mapping;
  a.n_tokens = n_tokens;
  a.gn = gn;
  a.hd = hd;
  a.dtype = dtype;
  return ic::launch_kv_append(a, static_cast<hipStream_t>(stream));
}

int ic_rope_kv_append(void *q, int64_t q_stride_token, int hn, const void *k_new, const void *v_new,
                      int64_t new_stride_token, void *k_pool, void *v_pool, int64_t pool_stride_block,
                      int64_t pool_stride_head, int64_t pool_stride_token, const int64_t *slot_mapping,
                      const int32_t *positions, const float *cos_table, const float *sin_table,
                      int64_t table_rows, int64_t n_tokens, int gn, int hd, int block_size,
                      int64_t num_blocks, int dtype, void *stream) {
  if (n_tokens < 0 || table_rows <= 0 || hd <= 0 || hd % 2 != 0) return IC_ERR_BAD_SHAPE;
  if (!dtype_ok(dtype)) return IC_ERR_UNSUPPORTED;
  const int es = ic::elem_size(dtype);
  if ((hd * es) % 16 != 0) return IC_ERR_UNSUPPORTED;
  const bool has_kv = k_new != nullptr || v_new != nullptr;
  if (has_kv) {
    if (int rc = check_pool(pool_stride_block, pool_stride_head, pool_stride_token, gn, hd, block_size,
                            num_blocks, es))
      return rc;
  }
  if (q != nullptr && hn <= 0) return IC_ERR_BAD_SHAPE;
  if (n_tokens == 0) return IC_OK;
  if (!positions || !cos_table || !sin_table) return IC_ERR_NULL_POINTER;
  if (q == nullptr && !has_kv) return IC_ERR_NULL_POINTER;
  if (!aligned16(cos_table) || !aligned16(sin_table)) return IC_ERR_ALIGNMENT;
  if (q != nullptr) {
    if (q_stride_token < (int64_t)hn * hd) return IC_ERR_BAD_SHAPE;
    if (!aligned16(q) || !stride16(q_stride_token, es)) return IC_ERR_ALIGNMENT;
  }
  if (has_kv) {
    if (!k_new || !v_new || !k_pool || !v_pool || !slot_mapping) return IC_ERR_NULL_POINTER;
    if (new_stride_token < (int64_t)gn * hd) return IC_ERR_BAD_SHAPE;
    if (!aligned16(k_new) || !aligned16(v_new) || !aligned16(k_pool) || !aligned16(v_pool) ||
        !stride16(new_stride_token, es))
      return IC_ERR_ALIGNMENT;
  }
  ic::RopeAppendArgs a;
  a.append.k_new = k_new;
  a.append.v_new = v_new;
  a.append.new_stride_token = new_stride_token;
  a.append.k_pool = k_pool;
  a.append.v_pool = v_pool;
  a.append.pool = {pool_stride_block, pool_stride_head, pool_stride_token, has_kv ? num_blocks : 0,
                   has_kv ? block_size : 1};
  a.append.slot_mapping = slot_mapping;
  a.append.n_tokens = n_tokens;
  a.append.gn = gn;
  a.append.hd = hd;
  a.append.dtype = dtype;
  a.q = q;
  a.q_stride_token = q_stride_token;
  a.hn = hn;
  a.positions = positions;
  a.cos_table = cos_table;
  a.sin_table = sin_table;
  a.table_rows = table_rows;
  return ic::launch_rope_kv_append(a, static_cast<hipStream_t>(stream));
}

size_t ic_paged_decode_workspace_bytes(int n_seqs, int hn, int gn, int hd) {
  return ic_paged_decode_shared_workspace_bytes(n_seqs, hn, gn, hd, 1);
}

size_t ic_paged_decode_shared_workspace_bytes(int n_seqs, int hn, int gn, int hd, int cohort_size) {
  if (n_seqs <= 0 || hn <= 0 || gn <= 0 || hn % gn != 0 || hd <= 0 || cohort_size < 1) return 0;
  if (!ic::decode_layout(n_seqs, hn, gn, cohort_size).ok) return 0;
  return ic::decode_workspace(n_seqs, hn, gn, hd, cohort_size).total();
}

int ic_paged_decode(void *out, int64_t out_stride_seq, const void *q, int64_t q_stride_seq,
                    const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                    int64_t pool_stride_head, int64_t pool_stride_token, const int32_t *block_tables,
                    int64_t block_table_stride, const int32_t *context_lens, int n_seqs, int hn,
                    int gn, int hd, int block_size, int64_t num_blocks, int max_context_len,
                    float scale, int min_chunk_tokens, void *workspace, size_t workspace_bytes,
                    int dtype, void *stream) {
  return ic_paged_decode_shared(out, out_stride_seq, q, q_stride_seq, k_pool, v_pool, pool_stride_block,
                                pool_stride_head, pool_stride_token, block_tables, block_table_stride,
                                context_lens, n_seqs, hn, gn, hd, block_size, num_blocks,
                                max_context_len, scale, min_chunk_tokens, 1, nullptr, workspace,
                                workspace_bytes, dtype, stream);
}

int ic_paged_decode_shared(void *out, int64_t out_stride_seq, const void *q, int64_t q_stride_seq,
                           const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                           int64_t pool_stride_head, int64_t pool_stride_token,
                           const int32_t *block_tables, int64_t block_table_stride,
                           const int32_t *context_lens, int n_seqs, int hn, int gn, int hd,
                           int block_size, int64_t num_blocks, int max_context_len, float scale,
                           int min_chunk_tokens, int cohort_size, const int32_t *cohort_shared_blocks,
                           void *workspace, size_t workspace_bytes, int dtype, void *stream) {
  return decode_checked(out, out_stride_seq, q, q_stride_seq, k_pool, v_pool, pool_stride_block,
                        pool_stride_head, pool_stride_token, block_tables, block_table_stride,
                        context_lens, n_seqs, hn, gn, hd, block_size, num_blocks, max_context_len,
                        scale, min_chunk_tokens, cohort_size, cohort_shared_blocks, workspace,
                        workspace_bytes, ic::kMaxDecodeWaves, dtype, stream);
}

size_t ic_paged_decode_static_scratch_bytes(int n_seqs, int hn, int gn, int hd) {
  if (n_seqs <= 0 || hn <= 0 || gn <= 0 || hn % gn != 0 || hd <= 0) return 0;
  return ic::decode_workspace(n_seqs, hn, gn, hd, 1, kStaticMaxWaves).total();
}

int ic_paged_decode_static(void *out, int64_t out_stride_seq, const void *q, int64_t q_stride_seq,
                           const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                           int64_t pool_stride_head, int64_t pool_stride_token,
                           const int32_t *block_tables, int64_t block_table_stride,
                           const int32_t *context_lens, int n_seqs, int hn, int gn, int hd,
                           int block_size, int64_t num_blocks, int max_context_len, float scale,
                           int min_chunk_tokens, int dtype, void *stream) {
  if (n_seqs < 0 || hn <= 0 || gn <= 0 || hn % gn != 0 || hd <= 0) return IC_ERR_BAD_SHAPE;
  size_t need = 0;
  if (n_seqs > 0) {
    need = ic_paged_decode_static_scratch_bytes(n_seqs, hn, gn, hd);
    if (need == 0 || need > (size_t)IC_STATIC_SCRATCH_BYTES) return IC_ERR_STATIC_LIMIT;
  }
  void *ws = n_seqs > 0 ? static_scratch() : nullptr;  // an empty batch launches nothing
  if (n_seqs > 0 && ws == nullptr) return IC_ERR_LAUNCH;
  // Nothing in the workspace has to start at zero: the main kernel writes the prefix sums and
  // every partial the reduce pass reads, so a previous call's leftovers are never looked at.
  return decode_checked(out, out_stride_seq, q, q_stride_seq, k_pool, v_pool, pool_stride_block,
                        pool_stride_head, pool_stride_token, block_tables, block_table_stride,
                        context_lens, n_seqs, hn, gn, hd, block_size, num_blocks, max_context_len,
                        scale, min_chunk_tokens, 1, nullptr, ws, (size_t)IC_STATIC_SCRATCH_BYTES,
                        kStaticMaxWaves, dtype, stream);
}

int ic_paged_prefill(void *out, int64_t out_stride_token, const void *q, int64_t q_stride_token,
                     const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                     int64_t pool_stride_head, int64_t pool_stride_token,
                     const int32_t *block_tables, int64_t block_table_stride,
                     const int32_t *context_lens, const int32_t *cu_seqlens_q, int n_seqs,
                     int max_chunk_len, int hn, int gn, int hd, int block_size, int64_t num_blocks,
                     float scale, int causal, int dtype, void *stream) {
  return prefill_checked(out, out_stride_token, q, q_stride_token, k_pool, v_pool, pool_stride_block,
                         pool_stride_head, pool_stride_token, block_tables, block_table_stride,
                         context_lens, cu_seqlens_q, n_seqs, max_chunk_len, hn, gn, hd, block_size,
                         num_blocks, scale, causal, nullptr, 0, 0, 0, 0, dtype, stream);
}

int ic_paged_prefill_masked(void *out, int64_t out_stride_token, const void *q, int64_t q_stride_token,
                            const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                            int64_t pool_stride_head, int64_t pool_stride_token,
                            const int32_t *block_tables, int64_t block_table_stride,
                            const int32_t *context_lens, const int32_t *cu_seqlens_q, int n_seqs,
                            int max_chunk_len, int hn, int gn, int hd, int block_size,
                            int64_t num_blocks, float scale, const uint8_t *mask,
                            int64_t mask_stride_seq, int64_t mask_stride_head, int64_t mask_stride_row,
                            int64_t mask_keys, int dtype, void *stream) {
  if (n_seqs > 0 && max_chunk_len > 0 && mask == nullptr) return IC_ERR_NULL_POINTER;
  if (mask_stride_seq < 0 || mask_stride_head < 0 || mask_stride_row < 0 || mask_keys < 0) return IC_ERR_BAD_SHAPE;
  if (mask_stride_row != 0 && mask_stride_row < mask_keys) return IC_ERR_BAD_SHAPE;
  if (n_seqs > 0 && max_chunk_len > 0 && mask_keys < 1) return IC_ERR_BAD_SHAPE;  // a mask row holds a byte at least
  return prefill_checked(out, out_stride_token, q, q_stride_token, k_pool, v_pool, pool_stride_block,
                         pool_stride_head, pool_stride_token, block_tables, block_table_stride,
                         context_lens, cu_seqlens_q, n_seqs, max_chunk_len, hn, gn, hd, block_size,
                         num_blocks, scale, 0, mask, mask_stride_seq, mask_stride_head, mask_stride_row,
                         mask_keys, dtype, stream);
}

int ic_paged_decode_masked(void *out, int64_t out_stride_seq, const void *q, int64_t q_stride_seq,
                           const void *k_pool, const void *v_pool, int64_t pool_stride_block,
                           int64_t pool_stride_head, int64_t pool_stride_token,
                           const int32_t *block_tables, int64_t block_table_stride,
                           const int32_t *context_lens, int n_seqs, int hn, int gn, int hd,
                           int block_size, int64_t num_blocks, int max_context_len, float scale,
                           int min_chunk_tokens, const uint8_t *key_mask, int64_t key_mask_stride_seq,
                           int64_t key_mask_stride_head, void *workspace, size_t workspace_bytes,
                           int dtype, void *stream) {
  if (n_seqs > 0 && key_mask == nullptr) return IC_ERR_NULL_POINTER;
  return decode_checked(out, out_stride_seq, q, q_stride_seq, k_pool, v_pool, pool_stride_block,
                        pool_stride_head, pool_stride_token, block_tables, block_table_stride,
                        context_lens, n_seqs, hn, gn, hd, block_size, num_blocks, max_context_len,
                        scale, min_chunk_tokens, 1, nullptr, workspace, workspace_bytes,
                        ic::kMaxDecodeWaves, dtype, stream, key_mask, key_mask_stride_seq,
                        key_mask_stride_head);
}

}  // extern "C"
