// Shared device helpers for the gfx950 kernels: vector types, bf16/e4m3 conversion with
// explicit rounding points, wave64 reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "../../include/dsx.h"

namespace dsx {

// Host-side set-up that has to happen once on every device the library is used on (kernel attributes, device
// properties): `init` runs with that device current, under a lock, until it has succeeded once.
constexpr int kMaxDevices = 64;
struct PerDeviceOnce {
  std::mutex lock;
  bool done[kMaxDevices] = {};
};
template <class F>
inline int per_device_once(PerDeviceOnce& once, F&& init) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return DSX_EARCH;
  std::lock_guard<std::mutex> guard(once.lock);
  if (once.done[dev]) return DSX_OK;
  const int rc = init(dev);
  if (rc == DSX_OK) once.done[dev] = true;
  return rc;
}

// Compute units of the current device (0 when it cannot be asked).
inline int device_cus() {
  static PerDeviceOnce once;
  static int cus[kMaxDevices];
  int dev = -1;
  const int rc = per_device_once(once, [&](int d) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, d) != hipSuccess) return (int)DSX_EARCH;
    cus[d] = prop.multiProcessorCount;
    return (int)DSX_OK;
  });
  if (rc != DSX_OK || hipGetDevice(&dev) != hipSuccess) return 0;
  return cus[dev];
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// fp32 -> bf16 bits, round-to-nearest-even, NaN kept quiet (same result as torch's cast).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

// Two fp32 -> packed bf16 pair with the hardware converter (v_cvt_pk_bf16_f32, RNE).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

// Round an fp32 value to the nearest bf16 and return it widened again (an in-register
// "rounding point" reproducing an intermediate bf16 tensor of the torch op sequence): the hardware
// converter and a shift, two instructions where the integer formulation takes seven.
__device__ __forceinline__ float round_bf16(float f) { return __uint_as_float(pack_bf16x2(f, f) << 16); }
// Two roundings through one conversion: three instructions for the pair instead of four.
__device__ __forceinline__ void round_bf16_pair(float& a, float& b) {
  const uint32_t w = pack_bf16x2(a, b);
  a = __uint_as_float(w << 16);
  b = __uint_as_float(w & 0xffff0000u);
}

// The same, with the conversion kept as ONE instruction: left to itself the compiler splits the pair into two
// single conversions (each with its own shift and mask) wherever the two halves are used apart.
__device__ __forceinline__ void round_bf16_pair_fused(float& a, float& b) {
  uint32_t w;
  asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w) : "v"(a), "v"(b));
  a = __uint_as_float(w << 16);
  b = __uint_as_float(w & 0xffff0000u);
}
// max(m, |a|, |b|) in one instruction (the compiler spends two more on canonicalising |a| and |b|).
__device__ __forceinline__ float max3_abs(float m, float a, float b) {
  float r;
  asm("v_max3_f32 %0, %1, |%2|, |%3|" : "=v"(r) : "v"(m), "v"(a), "v"(b));
  return r;
}

// Unpack the two bf16 halves of a 32-bit word.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> OCP e4m3fn, round-to-nearest-even, subnormals kept (step 2^-9), no saturation:
// |v| >= 480 (everything that does not round to <= 448) and NaN give 0x7f | sign, like
// torch.Tensor.to(torch.float8_e4m3fn).
__device__ __forceinline__ uint32_t f32_to_e4m3_bits(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t sign = (u >> 24) & 0x80u;
  u &= 0x7fffffffu;
  uint32_t r;
  if (u >= 0x43f00000u) {            // |f| >= 480 (incl. inf/NaN): not representable
    r = 0x7fu;
  } else if (u < 0x3c800000u) {      // |f| < 2^-6: subnormal range, quantum 2^-9
    // adding 2^14 aligns the quantum 2^-9 with the fp32 ulp at 2^14 (2^-9); the FPU rounds RNE
    float t = __uint_as_float(u) + 16384.0f;
    r = __float_as_uint(t) - 0x46800000u;
  } else {
    uint32_t odd = (u >> 20) & 1u;
    u += ((uint32_t)(7 - 127) << 23) + 0x7ffffu + odd;   // re-bias and round mantissa to 3 bits
    r = u >> 20;
  }
  return r | sign;
}

__device__ __forceinline__ float e4m3_bits_to_f32(uint32_t b) {
  uint32_t sign = (b & 0x80u) << 24;
  uint32_t em = b & 0x7fu;
  float v;
  if (em == 0x7fu) {
    v = __uint_as_float(0x7fc00000u);
  } else if (em < 8u) {
    v = (float)em * 0.001953125f;  // subnormal: m * 2^-9
  } else {
    v = __uint_as_float((em << 20) + ((uint32_t)(127 - 7) << 23));
  }
  return __uint_as_float(__float_as_uint(v) | sign);
}

// Wavefront-wide butterfly reductions (every lane ends with the result).  Steps 32 and 16 use the gfx950
// lane-swap instructions, steps 8..1 fold a DPP row rotate / quad permute into the add or max itself: six
// short VALU instructions instead of six trips through the LDS crossbar (ds_bpermute).  Same pairing, same
// order (32, 16, 8, 4, 2, 1) and therefore the same fp32 result as the xor butterfly.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, false));
}
constexpr int kDppRowRor8 = 0x128, kDppRowRor4 = 0x124, kDppQuadXor2 = 0x4e, kDppQuadXor1 = 0xb1;

__device__ __forceinline__ float wave_max(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
  v = fmaxf(v, dpp_f32<kDppRowRor8>(v));
  v = fmaxf(v, dpp_f32<kDppRowRor4>(v));
  v = fmaxf(v, dpp_f32<kDppQuadXor2>(v));
  v = fmaxf(v, dpp_f32<kDppQuadXor1>(v));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(b[0]) + __uint_as_float(b[1]);
  v += dpp_f32<kDppRowRor8>(v);
  v += dpp_f32<kDppRowRor4>(v);
  v += dpp_f32<kDppQuadXor2>(v);
  v += dpp_f32<kDppQuadXor1>(v);
  return v;
}

// tanh-GELU in fp32 with the expression torch evaluates for approximate="tanh":
// 0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 x^3))).  tanh(u) = 1 - 2/(exp(2u)+1) has an
// absolute error of about one fp32 ulp of 1.0, like a library tanhf, and saturates to +-1 cleanly.
// Four fp32 -> four OCP e4m3 bytes of one dword with the hardware converter (v_cvt_pk_fp8_f32, RNE,
// two values per instruction).  For |v| <= 448 the result equals f32_to_e4m3_bits; beyond that the
// converter's out-of-range result is the hardware's, so callers that must reproduce torch's bare cast
// (NaN from 465 on) use this only on values already scaled into range.
__device__ __forceinline__ uint32_t pack_e4m3x4_inrange(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return (uint32_t)w;
}

__device__ __forceinline__ float gelu_tanh_f32(float x) {
  // 0.5 x (1 + tanh(u)), u = sqrt(2/pi) (x + 0.044715 x^3), written as x / (1 + exp(-2u)): seven VALU
  // instructions (two transcendental), no cancellation in the negative tail, no overflow (x * 0 for
  // x -> -inf).  Agrees with torch's fp32 evaluation of the tanh form to within its own rounding noise.
  const float c1 = -2.0f * 1.4426950408889634f * 0.7978845608028654f;
  const float c3 = c1 * 0.044715f;
  const float a = x * __builtin_fmaf(x * x, c3, c1);  // -2u * log2(e)
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(a));
}

// Exactly rounded a*b + c*d with every operation rounded on its own (no FMA contraction), the
// result separate torch kernels produce.
__device__ __forceinline__ float mul_add_unfused(float a, float b, float c, float d) {
#pragma clang fp contract(off)
  const float p0 = a * b;
  const float p1 = c * d;
  return p0 + p1;
}
__device__ __forceinline__ float mul_then_add_unfused(float a, float b, float c) {
#pragma clang fp contract(off)
  const float p0 = a * b;
  return p0 + c;
}

}  // namespace dsx
