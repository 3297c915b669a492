// KV append: scatter new K/V rows into the block pool, bit for bit.
//
// The rows are what a transformer layer produced for the new tokens
// (reference: ironcore/models/transformer.py:88-98); the pool slot of row t is
// slot_mapping[t] = block*block_size + token_in_block.
//
// HBM-bound byte copy.  One lane moves one 16-byte chunk with a single
// dwordx4 load and store; a workgroup covers a contiguous run of chunks of one
// token row, so both the read of the new row and the write of each
// (head, token) segment are fully coalesced.  K and V go in the same launch
// (blockIdx.z).  Algorithmic traffic: 2 * n_tokens * gn * hd * elem bytes read
// and the same written, plus 8 bytes of slot index per token.
#include "ic_device.h"
#include "ic_internal.h"
#include "../../include/ironcore_paged.h"

namespace ic {

namespace {

constexpr int kAppendThreads = 256;

__global__ __launch_bounds__(kAppendThreads) void kv_append_kernel(
    const char *__restrict__ k_new, const char *__restrict__ v_new, int64_t new_stride_bytes,
    char *__restrict__ k_pool, char *__restrict__ v_pool, int64_t stride_block_bytes,
    int64_t stride_head_bytes, int64_t stride_token_bytes, const int64_t *__restrict__ slot_mapping,
    int chunks_per_head, int chunks_per_row, int block_size, int64_t num_slots) {
  const int64_t t = blockIdx.y;
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= num_slots) return;
  const int c = blockIdx.x * kAppendThreads + threadIdx.x;
  if (c >= chunks_per_row) return;
  const int64_t blk = slot / block_size;
  const int64_t off = slot - blk * block_size;
  const int head = c / chunks_per_head;
  const int within = c - head * chunks_per_head;
  const char *src = (blockIdx.z == 0 ? k_new : v_new) + t * new_stride_bytes + (int64_t)c * 16;
  char *dst = (blockIdx.z == 0 ? k_pool : v_pool) + blk * stride_block_bytes +
              head * stride_head_bytes + off * stride_token_bytes + (int64_t)within * 16;
  store16(dst, load16(src));
}

}  // namespace

int launch_kv_append(const AppendArgs &a, hipStream_t stream) {
  if (a.n_tokens == 0) return IC_OK;
  const int es = elem_size(a.dtype);
  const int chunks_per_head = a.hd * es / 16;
  const int chunks_per_row = chunks_per_head * a.gn;
  dim3 grid((chunks_per_row + kAppendThreads - 1) / kAppendThreads, (unsigned)a.n_tokens, 2);
  // gridDim.y is limited to 65535: walk longer appends in slices.
  const int64_t kMaxY = 65535;
  for (int64_t t0 = 0; t0 < a.n_tokens; t0 += kMaxY) {
    const int64_t n = (a.n_tokens - t0 < kMaxY) ? a.n_tokens - t0 : kMaxY;
    grid.y = (unsigned)n;
    hipLaunchKernelGGL(kv_append_kernel, grid, dim3(kAppendThreads), 0, stream,
                       (const char *)a.k_new + t0 * a.new_stride_token * es,
                       (const char *)a.v_new + t0 * a.new_stride_token * es,
                       a.new_stride_token * es, (char *)a.k_pool, (char *)a.v_pool,
                       a.pool.stride_block * es, a.pool.stride_head * es, a.pool.stride_token * es,
                       a.slot_mapping + t0, chunks_per_head, chunks_per_row, a.pool.block_size,
                       a.pool.num_blocks * a.pool.block_size);
  }
  return hipGetLastError() == hipSuccess ? IC_OK : IC_ERR_LAUNCH;
}

}  // namespace ic
