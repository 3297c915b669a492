// Device-side helpers shared by the gfx950 kernels: 16-byte vector access,
// element-type traits, DPP lane-group reductions.  wave64 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ic {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int kWave = 64;

struct alignas(16) Vec16 {
  uint32_t w[4];
};

__device__ __forceinline__ Vec16 load16(const void *p) {
  return *reinterpret_cast<const Vec16 *>(p);
}
__device__ __forceinline__ void store16(void *p, const Vec16 &v) {
  *reinterpret_cast<Vec16 *>(p) = v;
}

// ---- element traits ------------------------------------------------------
// EPL: elements in one 16-byte lane load.
// dot(): sum over the EPL element pairs of two 16-byte chunks, fp32
// accumulate.  widen(): chunk -> EPL floats.  narrow(): float -> element.

struct Bf16 {
  using type = __bf16;
  static constexpr int EPL = 8;
  static __device__ __forceinline__ float dot(const Vec16 &a, const Vec16 &b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a.w[i]),
                                            __builtin_bit_cast(bf16x2_t, b.w[i]), acc, false);
    return acc;
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b),
                                           acc, false);
  }
  static __device__ __forceinline__ void widen(const Vec16 &a, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __builtin_bit_cast(float, a.w[i] << 16);
      f[2 * i + 1] = __builtin_bit_cast(float, a.w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ type narrow(float x) { return static_cast<__bf16>(x); }
};

struct F16 {
  using type = _Float16;
  static constexpr int EPL = 8;
  static __device__ __forceinline__ float dot(const Vec16 &a, const Vec16 &b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a.w[i]),
                                   __builtin_bit_cast(f16x2_t, b.w[i]), acc, false);
    return acc;
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), acc, false);
  }
  static __device__ __forceinline__ void widen(const Vec16 &a, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f16x2_t h = __builtin_bit_cast(f16x2_t, a.w[i]);
      f[2 * i] = static_cast<float>(h.x);
      f[2 * i + 1] = static_cast<float>(h.y);
    }
  }
  static __device__ __forceinline__ type narrow(float x) { return static_cast<_Float16>(x); }
};

struct F32 {
  using type = float;
  static constexpr int EPL = 4;
  static __device__ __forceinline__ float dot(const Vec16 &a, const Vec16 &b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc = __builtin_fmaf(__builtin_bit_cast(float, a.w[i]), __builtin_bit_cast(float, b.w[i]), acc);
    return acc;
  }
  static __device__ __forceinline__ void widen(const Vec16 &a, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __builtin_bit_cast(float, a.w[i]);
  }
  static __device__ __forceinline__ type narrow(float x) { return x; }
};

// ---- lane-group all-reduce -------------------------------------------------
// Sum over aligned groups of LANES consecutive lanes; every lane of the group
// ends with the total.  Up to 16 lanes stays inside one DPP row (no LDS
// traffic); wider groups finish with ds_bpermute exchanges.

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}

constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;  // lane i <- lane 7-i within each 8
constexpr int kDppRowMirror = 0x140;      // lane i <- lane 15-i within each 16
constexpr int kDppRowRor4 = 0x124;        // lane i <- lane (i+4)%16 within each 16
constexpr int kDppRowRor8 = 0x128;        // lane i <- lane (i+8)%16 within each 16

template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
  static_assert(LANES == 1 || LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16 ||
                    LANES == 32 || LANES == 64,
                "lane group must be a power of two");
  if (LANES >= 2) x += dpp_f32<kDppQuadXor1>(x);
  if (LANES >= 4) x += dpp_f32<kDppQuadXor2>(x);
  if (LANES >= 8) x += dpp_f32<kDppRowHalfMirror>(x);
  if (LANES >= 16) x += dpp_f32<kDppRowMirror>(x);
  if (LANES >= 32) x += __shfl_xor(x, 16, kWave);
  if (LANES >= 64) x += __shfl_xor(x, 32, kWave);
  return x;
}

}  // namespace ic
