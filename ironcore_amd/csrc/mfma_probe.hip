// What the matrix cores sustain on this device: a loop of independent
// v_mfma_f32_32x32x16_bf16 whose operands never leave the registers, one wave
// per SIMD on every CU.  The chunked-prefill roofline is quoted against the
// vendor's 2.5 PFLOP/s (2.4 GHz x 256 CUs x 4 SIMDs x 1 024 flop/clk); under
// matrix load the part's power management holds a lower clock, and this kernel
// measures the rate that is actually there to be used.  bench.py times it for
// a second or two (the clock needs that long to settle) and reports the
// figure beside the nominal peak.  No memory traffic, no LDS, no vector work.
#include "ic_device.h"
#include "ic_internal.h"
#include "../../include/ironcore_paged.h"

namespace ic {
namespace {

constexpr int kProbeMfmaPerIter = 16;

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}
// two bf16 values of magnitude 0.25 .. 2 with random signs and mantissas: operands that toggle
// the datapath the way real activations do (identical or zero operands draw less power and
// overstate the sustainable clock)
__device__ __forceinline__ int probe_bf16x2(uint32_t seed) {
  const uint32_t h = probe_hash(seed);
  const uint32_t a = (h & 0x8000u) | ((125u + (h & 3u) % 3u) << 7) | ((h >> 2) & 0x7fu);
  const uint32_t b = ((h >> 16) & 0x8000u) | ((125u + ((h >> 18) & 3u) % 3u) << 7) | ((h >> 20) & 0x7fu);
  return (int)(a | (b << 16));
}

typedef __attribute__((ext_vector_type(4))) int i32x4_t;

__global__ __launch_bounds__(4 * kWave) void mfma_probe_kernel(int iters, float *sink) {
  const int tid = threadIdx.x + blockIdx.x * blockDim.x;
  f32x16_t c0 = {}, c1 = {}, c2 = {}, c3 = {};
  i32x4_t b, a[8];
  for (int i = 0; i < 4; ++i) b[i] = probe_bf16x2(tid * 4 + i + 99);
  for (int j = 0; j < 8; ++j)
    for (int i = 0; i < 4; ++i) a[j][i] = probe_bf16x2(tid * 64 + j * 4 + i);
  for (int it = 0; it < iters; ++it) {
    // four accumulators in turn (no MFMA waits for the one before it), eight A operands in
    // rotation (consecutive MFMAs see different data)
#define IC_PROBE_STEP(acc, areg) "v_mfma_f32_32x32x16_bf16 " acc ", " areg ", %12, " acc "\n"
    asm volatile(IC_PROBE_STEP("%0", "%4") IC_PROBE_STEP("%1", "%5") IC_PROBE_STEP("%2", "%6") IC_PROBE_STEP("%3", "%7")
                 IC_PROBE_STEP("%0", "%8") IC_PROBE_STEP("%1", "%9") IC_PROBE_STEP("%2", "%10") IC_PROBE_STEP("%3", "%11")
                 IC_PROBE_STEP("%0", "%5") IC_PROBE_STEP("%1", "%6") IC_PROBE_STEP("%2", "%7") IC_PROBE_STEP("%3", "%8")
                 IC_PROBE_STEP("%0", "%9") IC_PROBE_STEP("%1", "%10") IC_PROBE_STEP("%2", "%11") IC_PROBE_STEP("%3", "%4")
                 : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3), "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]),
                   "+v"(a[5]), "+v"(a[6]), "+v"(a[7])
                 : "v"(b));
#undef IC_PROBE_STEP
    if ((it & 1023) == 1023) {  // keep the sums finite
      // The compiler does not see the MFMAs inside the block above, so it cannot place the wait
      // states a vector read of their results needs: wait out more than the longest MFMA first.
      asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3));
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        c0[i] *= 1e-3f;
        c1[i] *= 1e-3f;
        c2[i] *= 1e-3f;
        c3[i] *= 1e-3f;
      }
    }
  }
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3));
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == 12345.678f) sink[0] = s;  // never true in practice: keeps the loop alive
}

}  // namespace

int64_t launch_mfma_probe(int iters, void *sink, hipStream_t stream) {
  const int wgs = device_cu_count();
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(wgs), dim3(4 * kWave), 0, stream, iters, static_cast<float *>(sink));
  if (hipGetLastError() != hipSuccess) return IC_ERR_LAUNCH;
  // flops of the launch: waves x iterations x MFMAs x 2 * 32 * 32 * 16
  return (int64_t)wgs * 4 * iters * kProbeMfmaPerIter * (2LL * 32 * 32 * 16);
}

}  // namespace ic
