// Bandwidth-bound row kernels of the DiT block: AdaLN modulate (LayerNorm + scale/shift),
// gated residual, tanh-GELU (optionally concatenated behind an untouched prefix), flow-match Euler
// update.  A wavefront (rows up to 6144 wide) or a workgroup of 256 threads owns one row, keeps it in
// registers (16-byte loads, 8 bf16 per chunk), reduces through the wavefront (plus a 4-entry LDS
// exchange for workgroup rows), and can emit the row as bf16 and/or as per-token-scaled e4m3 (the
// operand format of the following FP8 GEMM) in the same pass.
#include "common.h"

namespace dsx {

// Row reductions for TPR threads per row: TPR == 64 is one wavefront per row (four rows per
// workgroup, no LDS, no barrier); TPR == 128 is a pair of wavefronts per row (two rows per workgroup);
// TPR == 256 is the whole workgroup on one row.
template <int TPR>
__device__ __forceinline__ float row_sum(float v, float* red) {
  v = wave_sum(v);
  if (TPR == 64) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();  // protect `red` against a previous reduction still being read
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  if (TPR == 128) return red[w & 2] + red[w | 1];
  return red[0] + red[1] + red[2] + red[3];
}
template <int TPR>
__device__ __forceinline__ float row_max(float v, float* red) {
  v = wave_max(v);
  if (TPR == 64) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  if (TPR == 128) return fmaxf(red[w & 2], red[w | 1]);
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__device__ __forceinline__ void unpack8(const u32x4& w, float* v) {
  v[0] = bf16_lo(w.x); v[1] = bf16_hi(w.x); v[2] = bf16_lo(w.y); v[3] = bf16_hi(w.y);
  v[4] = bf16_lo(w.z); v[5] = bf16_hi(w.z); v[6] = bf16_lo(w.w); v[7] = bf16_hi(w.w);
}
__device__ __forceinline__ u32x4 pack8(const float* v) {
  u32x4 o;
  o.x = pack_bf16x2(v[0], v[1]);
  o.y = pack_bf16x2(v[2], v[3]);
  o.z = pack_bf16x2(v[4], v[5]);
  o.w = pack_bf16x2(v[6], v[7]);
  return o;
}
__device__ __forceinline__ u32x2 quant8(const float* v, float inv) {  // |v * inv| <= 448 by construction
  u32x2 r;
  r.x = pack_e4m3x4_inrange(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
  r.y = pack_e4m3x4_inrange(v[4] * inv, v[5] * inv, v[6] * inv, v[7] * inv);
  return r;
}

// Emit a row held as NCH register chunks of 8 already-bf16-rounded floats.
template <int NCH, int TPR>
__device__ __forceinline__ void emit_row(float (&val)[NCH][8], int nchunk, uint16_t* y, uint8_t* q,
                                         float* q_scale, int64_t row, float* red, bool live = true) {
  const int t = threadIdx.x % TPR;
  if (!live) nchunk = 0;  // a row slot past the last row takes part in the reductions' barriers, stores nothing
  if (y) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = t + i * TPR;
      if (c < nchunk) reinterpret_cast<u32x4*>(y)[c] = pack8(val[i]);
    }
  }
  if (q && !q_scale) {
    // the reference's bare cast (utils/fp8_linear.py:35): unit scale, what lies beyond e4m3's range becomes NaN
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = t + i * TPR;
      u32x2 r;
      r.x = f32_to_e4m3_bits(val[i][0]) | (f32_to_e4m3_bits(val[i][1]) << 8) | (f32_to_e4m3_bits(val[i][2]) << 16) |
            (f32_to_e4m3_bits(val[i][3]) << 24);
      r.y = f32_to_e4m3_bits(val[i][4]) | (f32_to_e4m3_bits(val[i][5]) << 8) | (f32_to_e4m3_bits(val[i][6]) << 16) |
            (f32_to_e4m3_bits(val[i][7]) << 24);
      if (c < nchunk) reinterpret_cast<u32x2*>(q)[c] = r;
    }
  } else if (q) {
    float amax = 0.f;  // slots past the end of the row hold zeros (callers see to that)
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
#pragma unroll
      for (int j = 0; j < 8; j += 2) amax = max3_abs(amax, val[i][j], val[i][j + 1]);
    }
    amax = fmaxf(row_max<TPR>(amax, red), 1e-12f);
    const float inv = 448.0f / amax;
    if (t == 0 && live) q_scale[row] = amax / 448.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = t + i * TPR;
      if (c < nchunk) reinterpret_cast<u32x2*>(q)[c] = quant8(val[i], inv);
    }
  }
}

template <int NCH, int TPR>
__global__ __launch_bounds__(256) void adaln_modulate_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint16_t* __restrict__ scale,
    const uint16_t* __restrict__ shift, int64_t mod_sb, int64_t rows_per_batch,
    const uint16_t* __restrict__ ln_w, const uint16_t* __restrict__ ln_b, float eps,
    uint16_t* __restrict__ y, int64_t ldy, uint8_t* __restrict__ q, int64_t ldq,
    float* __restrict__ q_scale, int64_t rows, int D) {
  __shared__ float red[4];
  const int t = threadIdx.x % TPR;
  int64_t row = (int64_t)blockIdx.x * (256 / TPR) + threadIdx.x / TPR;
  const bool live = row < rows;  // fails for whole row slots only (TPR < 256)
  if (!live) row = rows - 1;
  const int nchunk = D >> 3;
  // Chunk slots past the end of the row are clamped onto its last chunk, so that no load sits under a
  // lane predicate: the compiler then issues a row's loads back to back instead of waiting for each.
  int cc[NCH];
  bool ok[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = t + i * TPR;
    ok[i] = c < nchunk;
    cc[i] = min(c, nchunk - 1);
  }
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * ldx);
  const int64_t bidx = row / rows_per_batch;
  const u32x4* sc = scale ? reinterpret_cast<const u32x4*>(scale + bidx * mod_sb) : nullptr;
  const u32x4* sh = shift ? reinterpret_cast<const u32x4*>(shift + bidx * mod_sb) : nullptr;
  u32x4 raw[NCH], sraw[NCH], hraw[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) raw[i] = xr[cc[i]];
  // the modulation vectors are L2 hits (every row of a batch entry reads the same ones); fetched here, they
  // arrive under the two row reductions
  if (sc) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) sraw[i] = sc[cc[i]];
  }
  if (sh) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) hraw[i] = sh[cc[i]];
  }
  float val[NCH][8];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    unpack8(raw[i], val[i]);
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) part += val[i][j];
    sum += ok[i] ? part : 0.f;
  }
  const float mean = row_sum<TPR>(sum, red) / (float)D;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float d = val[i][j] - mean;
      part += d * d;
    }
    sq += ok[i] ? part : 0.f;
  }
  const float rstd = rsqrtf(row_sum<TPR>(sq, red) / (float)D + eps);
  const bool ragged = nchunk != NCH * TPR;  // uniform
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (val[i][j] - mean) * rstd;
    if (ln_w) {
      float w[8];
      unpack8(reinterpret_cast<const u32x4*>(ln_w)[cc[i]], w);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] *= w[j];
    }
    if (ln_b) {
      float bb[8];
      unpack8(reinterpret_cast<const u32x4*>(ln_b)[cc[i]], bb);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] += bb[j];
    }
    // every bf16 tensor of the separate ops is a rounding point: LayerNorm output, 1 + scale, the product,
    // the sum; roundings go in pairs through one conversion
#pragma unroll
    for (int j = 0; j < 8; j += 2) round_bf16_pair_fused(v[j], v[j + 1]);
    if (sc) {
      float s8[8];
      unpack8(sraw[i], s8);
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        float a = 1.0f + s8[j], b = 1.0f + s8[j + 1];
        round_bf16_pair_fused(a, b);
        v[j] *= a;
        v[j + 1] *= b;
        round_bf16_pair_fused(v[j], v[j + 1]);
      }
    }
    if (sh) {
      float h8[8];
      unpack8(hraw[i], h8);
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        v[j] += h8[j];
        v[j + 1] += h8[j + 1];
        round_bf16_pair_fused(v[j], v[j + 1]);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) val[i][j] = v[j];
  }
  if (ragged) {  // slots past the end of the row: a zero cannot raise the row's absmax
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) val[i][j] = ok[i] ? val[i][j] : 0.f;
  }
  if (!live && TPR == 64) return;  // wave-uniform; wider row slots share the workgroup's barriers
  emit_row<NCH, TPR>(val, nchunk, y ? y + row * ldy : nullptr, q ? q + row * ldq : nullptr, q_scale, row,
                     red, live);
}

// The form of adaln_modulate_kernel<NCH, 64> the DiT step launches a hundred times: rows of exactly NCH * 512
// values, both modulation vectors, no LayerNorm affine, e4m3 output with its per-token scale and nothing else.  With
// every option fixed at compile time the row is one straight line of code; the arithmetic and its order are those of
// the general kernel (same bits out).
template <int NCH>
__global__ __launch_bounds__(256) void adaln_quant_rows_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint16_t* __restrict__ scale,
    const uint16_t* __restrict__ shift, int64_t mod_sb, int64_t rows_per_batch, float eps,
    uint8_t* __restrict__ q, int64_t ldq, float* __restrict__ q_scale, int64_t rows) {
  const int t = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;  // wave-uniform; the kernel has no barrier
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * ldx);
  const int64_t bidx = row / rows_per_batch;
  const u32x4* sc = reinterpret_cast<const u32x4*>(scale + bidx * mod_sb);
  const u32x4* sh = reinterpret_cast<const u32x4*>(shift + bidx * mod_sb);
  u32x4 raw[NCH], sraw[NCH], hraw[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) raw[i] = xr[t + i * 64];
#pragma unroll
  for (int i = 0; i < NCH; ++i) sraw[i] = sc[t + i * 64];
#pragma unroll
  for (int i = 0; i < NCH; ++i) hraw[i] = sh[t + i * 64];
  float val[NCH][8];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    unpack8(raw[i], val[i]);
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) part += val[i][j];
    sum += part;
  }
  const float mean = wave_sum(sum) / (float)(NCH * 512);
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      val[i][j] -= mean;
      part += val[i][j] * val[i][j];
    }
    sq += part;
  }
  const float rstd = rsqrtf(wave_sum(sq) / (float)(NCH * 512) + eps);
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float s8[8], h8[8];
    unpack8(sraw[i], s8);
    unpack8(hraw[i], h8);
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      float v0 = val[i][j] * rstd, v1 = val[i][j + 1] * rstd;
      round_bf16_pair_fused(v0, v1);
      float a = 1.0f + s8[j], b = 1.0f + s8[j + 1];
      round_bf16_pair_fused(a, b);
      v0 *= a;
      v1 *= b;
      round_bf16_pair_fused(v0, v1);
      v0 += h8[j];
      v1 += h8[j + 1];
      round_bf16_pair_fused(v0, v1);
      val[i][j] = v0;
      val[i][j + 1] = v1;
      amax = max3_abs(amax, v0, v1);
    }
  }
  amax = fmaxf(wave_max(amax), 1e-12f);
  const float inv = 448.0f / amax;
  if (t == 0) q_scale[row] = amax / 448.0f;
  u32x2* qr = reinterpret_cast<u32x2*>(q + row * ldq);
#pragma unroll
  for (int i = 0; i < NCH; ++i) qr[t + i * 64] = quant8(val[i], inv);
}

// RMSNorm over the whole row followed by an optional per-head RoPE (head dim 128, pairs (2i, 2i+1)):
//   y = bf16( bf16(x * rsqrt(mean(x^2) + eps)) * w ),  then  (c y0 - s y1, s y0 + c y1) -> bf16.
// The row is a token's full model dim (Wan normalises q and k over all heads at once).
template <int NCH, int TPR>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                           const uint16_t* __restrict__ w, float eps,
                                                           const float* __restrict__ rope, int64_t rope_sb,
                                                           int64_t rows_per_batch, uint16_t* __restrict__ out,
                                                           int64_t ldo, int64_t rows, int D,
                                                           float* head_norm2_max) {
  __shared__ float red[4];
  const int t = threadIdx.x % TPR;
  int64_t row = (int64_t)blockIdx.x * (256 / TPR) + threadIdx.x / TPR;
  const bool live = row < rows;
  if (!live) row = rows - 1;
  const int nchunk = D >> 3;
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * ldx);
  // slots past the end of the row are clamped onto its last chunk: no load sits under a lane predicate
  int cc[NCH];
  bool ok[NCH];
  u32x4 raw[NCH], wraw[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = t + i * TPR;
    ok[i] = c < nchunk;
    cc[i] = min(c, nchunk - 1);
    raw[i] = xr[cc[i]];
  }
#pragma unroll
  for (int i = 0; i < NCH; ++i) wraw[i] = reinterpret_cast<const u32x4*>(w)[cc[i]];
  float val[NCH][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    unpack8(raw[i], val[i]);
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) part += val[i][j] * val[i][j];
    ss += ok[i] ? part : 0.f;
  }
  const float rrms = rsqrtf(row_sum<TPR>(ss, red) / (float)D + eps);
  float hmax = 0.f;
  if (live) {  // wave-uniform
    const float* rp = rope ? rope + (row / rows_per_batch) * rope_sb + (row % rows_per_batch) * 128 : nullptr;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      float wv[8];
      unpack8(wraw[i], wv);
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = round_bf16(round_bf16(val[i][j] * rrms) * wv[j]);
      if (rp) {
        const int off = (cc[i] * 8) & 127;  // offset inside the head: floats (cos, sin) of pairs off/2 .. off/2+3
        const f32x4 t0 = *reinterpret_cast<const f32x4*>(rp + off);
        const f32x4 t1 = *reinterpret_cast<const f32x4*>(rp + off + 4);
        const float cs[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float co = cs[2 * k], sn = cs[2 * k + 1];
          const float x0 = v[2 * k], x1 = v[2 * k + 1];
          v[2 * k] = mul_add_unfused(co, x0, -sn, x1);
          v[2 * k + 1] = mul_add_unfused(sn, x0, co, x1);
        }
      }
      if (ok[i]) reinterpret_cast<u32x4*>(out + row * ldo)[cc[i]] = pack8(v);
      if (head_norm2_max) {  // uniform
        // a 128-wide head is 16 chunks = the 16 lanes of one DPP row (TPR is a multiple of 16)
        float n2 = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) n2 += v[j] * v[j];
        n2 = ok[i] ? n2 : 0.f;
        n2 += dpp_f32<kDppRowRor8>(n2);
        n2 += dpp_f32<kDppRowRor4>(n2);
        n2 += dpp_f32<kDppQuadXor2>(n2);
        n2 += dpp_f32<kDppQuadXor1>(n2);
        hmax = fmaxf(hmax, n2);
      }
    }
  }
  if (head_norm2_max) {
    // One look at the current maximum per workgroup, one atomic only when it has to rise.  The look is a
    // device-scope load (the eight L2s do not see each other's atomics otherwise) and the value only ever
    // grows, so a stale look costs one redundant atomic and nothing else.  Non-negative floats order like
    // their bit patterns; +Inf stays the maximum once seen.
    hmax = wave_max(hmax);
    const int w = threadIdx.x >> 6;
    __syncthreads();  // `red` may still be read by the row sum of a slower wave
    if ((threadIdx.x & 63) == 0) red[w] = hmax;
    __syncthreads();
    if (threadIdx.x == 0) {  // (waves of rows past the end bring 0)
      hmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
      const float seen = __hip_atomic_load(head_norm2_max, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (!(hmax <= seen)) atomicMax(reinterpret_cast<unsigned int*>(head_norm2_max), __float_as_uint(hmax));
    }
  }
}

// erf-GELU as torch evaluates nn.GELU() in fp32: x * 0.5 * (1 + erf(x / sqrt(2))).
__device__ __forceinline__ float gelu_erf_f32(float x) { return x * 0.5f * (1.0f + erff(x * 0.70710678118654752f)); }

// GELU (tanh form, or the erf form with ERF) of x, optionally preceded in the OUTPUT row by an unmodified prefix:
// out row = [ prefix (Dp) | gelu(x) (D) ].  The prefix form is the single-stream block's
// cat([attention, gelu(mlp)]) built directly in the operand format of proj_out.
template <int NCH, bool ERF>
__global__ __launch_bounds__(256) void gelu_tanh_kernel(const uint16_t* __restrict__ prefix, int64_t ldp,
                                                        int Dp, const uint16_t* __restrict__ x, int64_t ldx,
                                                        uint16_t* __restrict__ y, int64_t ldy,
                                                        uint8_t* __restrict__ q, int64_t ldq,
                                                        float* __restrict__ q_scale, int D) {
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int npre = Dp >> 3;
  const int nchunk = npre + (D >> 3);
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * ldx);
  const u32x4* pr = reinterpret_cast<const u32x4*>(prefix + row * ldp);
  // slots past the end of the row are clamped onto its last chunk: no load sits under a lane predicate
  u32x4 raw[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = min(tid + i * 256, nchunk - 1);
    raw[i] = __builtin_nontemporal_load(c < npre ? pr + c : xr + (c - npre));
  }
  float val[NCH][8];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = tid + i * 256;
    unpack8(raw[i], val[i]);
    if (c >= npre) {
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        val[i][j] = ERF ? gelu_erf_f32(val[i][j]) : gelu_tanh_f32(val[i][j]);
        val[i][j + 1] = ERF ? gelu_erf_f32(val[i][j + 1]) : gelu_tanh_f32(val[i][j + 1]);
        round_bf16_pair_fused(val[i][j], val[i][j + 1]);
      }
    }
    if (c >= nchunk) {
#pragma unroll
      for (int j = 0; j < 8; ++j) val[i][j] = 0.f;  // keeps the row's absmax untouched
    }
  }
  emit_row<NCH, 256>(val, nchunk, y ? y + row * ldy : nullptr, q ? q + row * ldq : nullptr, q_scale, row,
                     red);
}

__global__ __launch_bounds__(256) void gated_residual_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint16_t* __restrict__ yv, int64_t ldy,
    const uint16_t* __restrict__ gate, int64_t gate_sb, int64_t rows_per_batch,
    uint16_t* __restrict__ out, int64_t ldo, int64_t rows, int D) {
  const int nchunk = D >> 3;
  const int64_t total = rows * nchunk;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; id < total; id += stride) {
    const int64_t row = id / nchunk;
    const int c = (int)(id - row * nchunk);
    float a[8], b[8];
    unpack8(*reinterpret_cast<const u32x4*>(x + row * ldx + c * 8), a);
    unpack8(*reinterpret_cast<const u32x4*>(yv + row * ldy + c * 8), b);
    if (gate) {
      float gt[8];
      unpack8(*reinterpret_cast<const u32x4*>(gate + (row / rows_per_batch) * gate_sb + c * 8), gt);
#pragma unroll
      for (int j = 0; j < 8; ++j) b[j] = round_bf16(gt[j] * b[j]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) a[j] = a[j] + b[j];
    *reinterpret_cast<u32x4*>(out + row * ldo + c * 8) = pack8(a);
  }
}

template <bool FP32>
__global__ __launch_bounds__(256) void euler_step_kernel(const void* __restrict__ lat,
                                                         const void* __restrict__ v, float dt,
                                                         void* __restrict__ out, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    if (FP32) {
      const float a = reinterpret_cast<const float*>(lat)[i];
      const float b = reinterpret_cast<const float*>(v)[i];
      reinterpret_cast<float*>(out)[i] = mul_then_add_unfused(b, dt, a);
    } else {
      const float a = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(lat)[i]);
      const float b = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(v)[i]);
      // `model_outputs * dt` is a bf16 tensor, the sum is taken in fp32 and rounded once
      const float prod = round_bf16(b * dt);
      reinterpret_cast<uint16_t*>(out)[i] = (uint16_t)f32_to_bf16_bits(a + prod);
    }
  }
}

static inline bool misaligned16(const void* p) { return ((uintptr_t)p & 15) != 0; }

}  // namespace dsx

extern "C" int dsx_adaln_modulate(const void* x, int64_t ldx, const void* scale, const void* shift,
                                  int64_t mod_sb, int64_t rows_per_batch, const void* ln_w,
                                  const void* ln_b, float eps, void* y, int64_t ldy, void* q,
                                  int64_t ldq, float* q_scale, int64_t rows, int64_t D,
                                  void* stream) {
  using namespace dsx;
  if (rows == 0) return DSX_OK;  // an empty batch has no buffers to point at
  if (!x || (!y && !q)) return DSX_ENULL;
  if (rows < 0 || D <= 0 || (D & 7) || D > 16384 || ldx < D || (y && ldy < D) || (q && ldq < D) ||
      rows_per_batch <= 0)
    return DSX_EBADSHAPE;
  if ((ldx & 7) || (y && (ldy & 7)) || (q && (ldq & 7)) || (mod_sb & 7) || misaligned16(x) ||
      misaligned16(y) || ((uintptr_t)q & 7) || misaligned16(scale) || misaligned16(shift) ||
      misaligned16(ln_w) || misaligned16(ln_b))
    return DSX_EALIGN;
  if (rows == 0) return DSX_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 block(256);
#define DSX_LAUNCH_ADALN(NCH, TPR)                                                                 \
  adaln_modulate_kernel<NCH, TPR><<<dim3((unsigned)((rows + 256 / TPR - 1) / (256 / TPR))), block, 0, st>>>( \
      (const uint16_t*)x, ldx, (const uint16_t*)scale, (const uint16_t*)shift, mod_sb,             \
      rows_per_batch, (const uint16_t*)ln_w, (const uint16_t*)ln_b, eps, (uint16_t*)y, ldy,        \
      (uint8_t*)q, ldq, q_scale, rows, (int)D)
  // One wavefront per row while a row fits 6 chunks per lane and there are rows enough to fill the chip.
  // Wider rows: 12 chunks per lane cost 217 registers, two waves per SIMD and 266 us for 32760 x 5120; a
  // workgroup per row takes 160-175 us, a pair of wavefronts per row (two rows per workgroup) 145-150 us.
  if (D == 512 * 6 && rows >= 1024 && scale && shift && !ln_w && !ln_b && q && q_scale && !y)
    adaln_quant_rows_kernel<6><<<dim3((unsigned)((rows + 3) / 4)), block, 0, st>>>(
        (const uint16_t*)x, ldx, (const uint16_t*)scale, (const uint16_t*)shift, mod_sb, rows_per_batch, eps,
        (uint8_t*)q, ldq, q_scale, rows);
  else if (D <= 512 * 6 && rows >= 1024) DSX_LAUNCH_ADALN(6, 64);
  else if (D <= 2048 * 2) DSX_LAUNCH_ADALN(2, 256);
  else if (D <= 1024 * 5 && rows >= 2048) DSX_LAUNCH_ADALN(5, 128);
  else if (D <= 2048 * 3) DSX_LAUNCH_ADALN(3, 256);
  else DSX_LAUNCH_ADALN(8, 256);
#undef DSX_LAUNCH_ADALN
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

static int launch_gelu(const void* prefix, int64_t ldp, int64_t Dp, const void* x, int64_t ldx, void* y,
                       int64_t ldy, void* q, int64_t ldq, float* q_scale, int64_t rows, int64_t D,
                       hipStream_t st, bool erf = false) {
  using namespace dsx;
  const int64_t Dt = Dp + D;
  dim3 grid((unsigned)rows), block(256);
#define DSX_LAUNCH_GELU(NCH, ERF)                                                                             \
  gelu_tanh_kernel<NCH, ERF><<<grid, block, 0, st>>>((const uint16_t*)prefix, ldp, (int)Dp, (const uint16_t*)x, \
                                                     ldx, (uint16_t*)y, ldy, (uint8_t*)q, ldq, q_scale, (int)D)
  if (erf) DSX_LAUNCH_GELU(8, true);  // (the erf form serves a 257-row embedder: one instantiation is enough)
  else if (Dt <= 2048 * 2) DSX_LAUNCH_GELU(2, false);
  else if (Dt <= 2048 * 6) DSX_LAUNCH_GELU(6, false);
  else DSX_LAUNCH_GELU(8, false);
#undef DSX_LAUNCH_GELU
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

static int gelu_plain(const void* x, int64_t ldx, void* y, int64_t ldy, void* q, int64_t ldq, float* q_scale,
                      int64_t rows, int64_t D, void* stream, bool erf) {
  using namespace dsx;
  if (rows == 0) return DSX_OK;  // an empty batch has no buffers to point at
  if (!x || (!y && !q)) return DSX_ENULL;
  if (rows < 0 || D <= 0 || (D & 7) || D > 16384 || ldx < D || (y && ldy < D) || (q && ldq < D))
    return DSX_EBADSHAPE;
  if ((ldx & 7) || (y && (ldy & 7)) || (q && (ldq & 7)) || misaligned16(x) || misaligned16(y) ||
      ((uintptr_t)q & 7))
    return DSX_EALIGN;
  return launch_gelu(x, 0, 0, x, ldx, y, ldy, q, ldq, q_scale, rows, D, (hipStream_t)stream, erf);
}

extern "C" int dsx_gelu_tanh(const void* x, int64_t ldx, void* y, int64_t ldy, void* q, int64_t ldq,
                             float* q_scale, int64_t rows, int64_t D, void* stream) {
  return gelu_plain(x, ldx, y, ldy, q, ldq, q_scale, rows, D, stream, false);
}

extern "C" int dsx_gelu_erf(const void* x, int64_t ldx, void* y, int64_t ldy, void* q, int64_t ldq,
                            float* q_scale, int64_t rows, int64_t D, void* stream) {
  return gelu_plain(x, ldx, y, ldy, q, ldq, q_scale, rows, D, stream, true);
}

extern "C" int dsx_concat_gelu_tanh(const void* prefix, int64_t ldp, int64_t Dp, const void* x, int64_t ldx,
                                    void* y, int64_t ldy, void* q, int64_t ldq, float* q_scale,
                                    int64_t rows, int64_t D, void* stream) {
  using namespace dsx;
  if (rows == 0) return DSX_OK;
  if (!prefix || !x || (!y && !q)) return DSX_ENULL;
  const int64_t Dt = Dp + D;
  if (rows < 0 || D <= 0 || Dp <= 0 || (D & 7) || (Dp & 7) || Dt > 16384 || ldx < D || ldp < Dp ||
      (y && ldy < Dt) || (q && ldq < Dt))
    return DSX_EBADSHAPE;
  if ((ldx & 7) || (ldp & 7) || (y && (ldy & 7)) || (q && (ldq & 7)) || misaligned16(x) ||
      misaligned16(prefix) || misaligned16(y) || ((uintptr_t)q & 7))
    return DSX_EALIGN;
  if (rows == 0) return DSX_OK;
  return launch_gelu(prefix, ldp, Dp, x, ldx, y, ldy, q, ldq, q_scale, rows, D, (hipStream_t)stream);
}

extern "C" int dsx_gated_residual(const void* x, int64_t ldx, const void* y, int64_t ldy,
                                  const void* gate, int64_t gate_sb, int64_t rows_per_batch,
                                  void* out, int64_t ldo, int64_t rows, int64_t D, void* stream) {
  using namespace dsx;
  if (rows == 0) return DSX_OK;
  if (!x || !y || !out) return DSX_ENULL;
  if (rows < 0 || D <= 0 || (D & 7) || D > (1 << 24) || ldx < D || ldy < D || ldo < D ||
      rows_per_batch <= 0)
    return DSX_EBADSHAPE;
  if ((ldx & 7) || (ldy & 7) || (ldo & 7) || (gate_sb & 7) || misaligned16(x) || misaligned16(y) ||
      misaligned16(out) || misaligned16(gate))
    return DSX_EALIGN;
  if (rows == 0) return DSX_OK;
  const int64_t total = rows * (D >> 3);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  gated_residual_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
      (const uint16_t*)x, ldx, (const uint16_t*)y, ldy, (const uint16_t*)gate, gate_sb,
      rows_per_batch, (uint16_t*)out, ldo, rows, (int)D);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

extern "C" int dsx_flow_match_euler_step(const void* latents, const void* v, float dt, void* out,
                                         int64_t n, int is_fp32, void* stream) {
  using namespace dsx;
  if (!latents || !v || !out) return DSX_ENULL;
  if (n < 0) return DSX_EBADSHAPE;
  if (n == 0) return DSX_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipStream_t st = (hipStream_t)stream;
  if (is_fp32)
    euler_step_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(latents, v, dt, out, n);
  else
    euler_step_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(latents, v, dt, out, n);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

extern "C" int dsx_rmsnorm_rows(const void* x, int64_t ldx, const void* w, float eps, const float* rope,
                                int64_t rope_sb, int64_t rows_per_batch, void* out, int64_t ldo, int64_t rows,
                                int64_t D, float* head_norm2_max, void* stream) {
  using namespace dsx;
  if (rows == 0) return DSX_OK;
  if (!x || !w || !out) return DSX_ENULL;
  if (rows < 0 || D <= 0 || (D & 7) || D > 16384 || ldx < D || ldo < D || rows_per_batch <= 0 ||
      ((rope || head_norm2_max) && (D & 127)))
    return DSX_EBADSHAPE;
  if ((ldx & 7) || (ldo & 7) || (rope_sb & 3) || misaligned16(x) || misaligned16(out) || misaligned16(w) ||
      misaligned16(rope) || ((uintptr_t)head_norm2_max & 3))
    return DSX_EALIGN;
  hipStream_t st = (hipStream_t)stream;
#define DSX_LAUNCH_RMS(NCH, TPR)                                                                           \
  rmsnorm_rows_kernel<NCH, TPR><<<dim3((unsigned)((rows + 256 / TPR - 1) / (256 / TPR))), dim3(256), 0, st>>>( \
      (const uint16_t*)x, ldx, (const uint16_t*)w, eps, rope, rope_sb, rows_per_batch, (uint16_t*)out, ldo,   \
      rows, (int)D, head_norm2_max)
  if (D <= 512 * 6 && rows >= 1024) DSX_LAUNCH_RMS(6, 64);
  else if (D > 4096 && D <= 1024 * 5 && rows >= 2048) DSX_LAUNCH_RMS(5, 128);  // as for AdaLN
  else if (D <= 2048 * 3) DSX_LAUNCH_RMS(3, 256);
  else DSX_LAUNCH_RMS(8, 256);
#undef DSX_LAUNCH_RMS
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}
