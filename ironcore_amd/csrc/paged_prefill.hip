// Chunked prefill against the block KV cache (MFMA path).
#include "ic_device.h"
#include "ic_internal.h"
#include "../../include/ironcore_paged.h"

namespace ic {

int launch_paged_prefill(const PrefillArgs &a, hipStream_t stream) {
  (void)a;
  (void)stream;
  return IC_ERR_UNSUPPORTED;
}

}  // namespace ic
