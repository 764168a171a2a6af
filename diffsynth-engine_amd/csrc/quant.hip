// bf16/fp32 -> e4m3 quantisation kernels (HBM-bound): per-token dynamic scale, per-tensor
// scaled cast, absmax.  One wave64 owns one row; rows are cached in registers between the
// absmax pass and the cast pass so every element is read from HBM once.
#include "common.h"

namespace dsx {

// Quantise 8 floats (already divided by the scale) to 8 e4m3 bytes.  IN_RANGE: every |v| <= 448
// (scaled quantisation), so the hardware converter applies.
template <bool IN_RANGE>
__device__ __forceinline__ u32x2 pack_e4m3x8(const float* v) {
  u32x2 r;
  if (IN_RANGE) {
    r.x = pack_e4m3x4_inrange(v[0], v[1], v[2], v[3]);
    r.y = pack_e4m3x4_inrange(v[4], v[5], v[6], v[7]);
    return r;
  }
  r.x = f32_to_e4m3_bits(v[0]) | (f32_to_e4m3_bits(v[1]) << 8) | (f32_to_e4m3_bits(v[2]) << 16) |
        (f32_to_e4m3_bits(v[3]) << 24);
  r.y = f32_to_e4m3_bits(v[4]) | (f32_to_e4m3_bits(v[5]) << 8) | (f32_to_e4m3_bits(v[6]) << 16) |
        (f32_to_e4m3_bits(v[7]) << 24);
  return r;
}

__device__ __forceinline__ void unpack_bf16x8(const u32x4& w, float* v) {
  v[0] = bf16_lo(w.x); v[1] = bf16_hi(w.x);
  v[2] = bf16_lo(w.y); v[3] = bf16_hi(w.y);
  v[4] = bf16_lo(w.z); v[5] = bf16_hi(w.z);
  v[6] = bf16_lo(w.w); v[7] = bf16_hi(w.w);
}

__device__ __forceinline__ float absmax_bf16x8(const u32x4& w) {
  // |bf16| compares like its bit pattern with the sign cleared
  float m = fabsf(bf16_lo(w.x));
  m = fmaxf(m, fabsf(bf16_hi(w.x)));
  m = fmaxf(m, fmaxf(fabsf(bf16_lo(w.y)), fabsf(bf16_hi(w.y))));
  m = fmaxf(m, fmaxf(fabsf(bf16_lo(w.z)), fabsf(bf16_hi(w.z))));
  m = fmaxf(m, fmaxf(fabsf(bf16_lo(w.w)), fabsf(bf16_hi(w.w))));
  return m;
}

// NCH: 16-byte chunks of the row cached per lane (row length <= NCH * 512 elements).
template <int NCH, bool SCALED>
__global__ __launch_bounds__(256) void quant_rowwise_kernel(const uint16_t* __restrict__ x,
                                                            int64_t ldx, uint8_t* __restrict__ q,
                                                            int64_t ldq,
                                                            float* __restrict__ scale_out,
                                                            int64_t M, int K) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int nchunk = K >> 3;
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * ldx);
  // slots past the end of the row are clamped onto its last chunk (a repeated chunk leaves the absmax as it
  // is), so that no load sits under a lane predicate and the row's loads are issued back to back
  u32x4 cache[NCH];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) cache[i] = __builtin_nontemporal_load(xr + min(lane + i * 64, nchunk - 1));
  if (SCALED) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) amax = fmaxf(amax, absmax_bf16x8(cache[i]));
  }
  float inv = 1.0f;
  if (SCALED) {
    amax = fmaxf(wave_max(amax), 1e-12f);
    inv = 448.0f / amax;
    if (lane == 0) scale_out[row] = amax / 448.0f;
  }
  u32x2* qr = reinterpret_cast<u32x2*>(q + row * ldq);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    int c = lane + i * 64;
    if (c < nchunk) {
      float v[8];
      unpack_bf16x8(cache[i], v);
      if (SCALED) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = v[j] * inv;
      }
      qr[c] = pack_e4m3x8<SCALED>(v);
    }
  }
}

template <bool FP32>
__global__ __launch_bounds__(256) void absmax_kernel(const void* __restrict__ x, int64_t n,
                                                     float* __restrict__ out) {
  float m = 0.f;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float v = FP32 ? reinterpret_cast<const float*>(x)[i]
                   : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(x)[i]);
    m = fmaxf(m, fabsf(v));
  }
  m = wave_max(m);
  // non-negative floats order like their bit patterns, so an integer max is exact
  if ((threadIdx.x & 63) == 0) atomicMax(reinterpret_cast<unsigned int*>(out), __float_as_uint(m));
}

template <bool FP32>
__global__ __launch_bounds__(256) void cast_scaled_kernel(const void* __restrict__ x,
                                                          const float* __restrict__ absmax,
                                                          float* __restrict__ scale_out,
                                                          uint8_t* __restrict__ q, int64_t n) {
  const bool scaled = absmax != nullptr;
  const float amax = scaled ? fmaxf(*absmax, 1e-12f) : 1.0f;
  const float inv = scaled ? 448.0f / amax : 1.0f;
  if (scaled && blockIdx.x == 0 && threadIdx.x == 0) *scale_out = amax / 448.0f;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float v = FP32 ? reinterpret_cast<const float*>(x)[i]
                   : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(x)[i]);
    if (scaled) v = v * inv;
    q[i] = (uint8_t)f32_to_e4m3_bits(v);
  }
}

template <bool SCALED>
static int launch_quant(const uint16_t* x, int64_t ldx, uint8_t* q, int64_t ldq, float* scale_out,
                        int64_t M, int K, hipStream_t st) {
  dim3 grid((unsigned)((M + 3) / 4)), block(256);
  if (K <= 512 * 2) {
    quant_rowwise_kernel<2, SCALED><<<grid, block, 0, st>>>(x, ldx, q, ldq, scale_out, M, K);
  } else if (K <= 512 * 6) {
    quant_rowwise_kernel<6, SCALED><<<grid, block, 0, st>>>(x, ldx, q, ldq, scale_out, M, K);
  } else if (K <= 512 * 10) {
    quant_rowwise_kernel<10, SCALED><<<grid, block, 0, st>>>(x, ldx, q, ldq, scale_out, M, K);
  } else if (K <= 512 * 24) {
    quant_rowwise_kernel<24, SCALED><<<grid, block, 0, st>>>(x, ldx, q, ldq, scale_out, M, K);
  } else if (K <= 512 * 32) {
    quant_rowwise_kernel<32, SCALED><<<grid, block, 0, st>>>(x, ldx, q, ldq, scale_out, M, K);
  } else {
    return DSX_EBADSHAPE;
  }
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

}  // namespace dsx

extern "C" int dsx_quant_fp8_rowwise(const void* x, int64_t ldx, void* q, int64_t ldq,
                                     float* scale_out, int64_t M, int64_t K, void* stream) {
  using namespace dsx;
  if (M == 0) return DSX_OK;  // an empty batch has no buffers to point at
  if (!x || !q) return DSX_ENULL;
  if (M < 0 || K <= 0 || (K & 7) || K > 512 * 32 || ldx < K || ldq < K) return DSX_EBADSHAPE;
  if ((ldx & 7) || (ldq & 7) || ((uintptr_t)x & 15) || ((uintptr_t)q & 7)) return DSX_EALIGN;
  if (M == 0) return DSX_OK;
  hipStream_t st = (hipStream_t)stream;
  if (scale_out)
    return launch_quant<true>((const uint16_t*)x, ldx, (uint8_t*)q, ldq, scale_out, M, (int)K, st);
  return launch_quant<false>((const uint16_t*)x, ldx, (uint8_t*)q, ldq, nullptr, M, (int)K, st);
}

extern "C" int dsx_absmax(const void* x, int64_t n, int is_fp32, float* absmax_out, void* stream) {
  using namespace dsx;
  if (!x || !absmax_out) return DSX_ENULL;
  if (n < 0) return DSX_EBADSHAPE;
  if (n == 0) return DSX_OK;
  hipStream_t st = (hipStream_t)stream;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  if (is_fp32)
    absmax_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(x, n, absmax_out);
  else
    absmax_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(x, n, absmax_out);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

extern "C" int dsx_cast_fp8_scaled(const void* x, int is_fp32, const float* absmax,
                                   float* scale_out, void* q, int64_t n, void* stream) {
  using namespace dsx;
  if (!x || !q || (absmax && !scale_out)) return DSX_ENULL;
  if (n < 0) return DSX_EBADSHAPE;
  if (n == 0) return DSX_OK;
  hipStream_t st = (hipStream_t)stream;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (is_fp32)
    cast_scaled_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(x, absmax, scale_out,
                                                                           (uint8_t*)q, n);
  else
    cast_scaled_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(x, absmax, scale_out,
                                                                            (uint8_t*)q, n);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}
