// Launchers shared between the attention translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/dsx.h"
#include "common.h"

namespace dsx {
// Attention without fused RMSNorm/RoPE (parameters already validated by dsx_attn_fwd).  `scratch` is
// optional device memory (16-byte aligned) for splitting the key range of the last round of workgroups.
int launch_attn_plain(const dsx_attn_params& p, void* scratch, int64_t scratch_bytes, hipStream_t stream);
// Scratch bytes with which launch_attn_plain would split (0 when it would not).
int64_t attn_plain_workspace_bytes(const dsx_attn_params& p);
// The same attention on the 16x16x32 MFMA shape (attn_plain16.hip), for launches of several full rounds of
// workgroups; whole units only (no key split, no fused q pre-processing).  launch_attn_plain decides.
int launch_attn_plain16(const dsx_attn_params& p, int64_t units, hipStream_t stream);
}  // namespace dsx

#ifdef __HIPCC__
namespace dsx {
// RMSNorm + RoPE on 8 consecutive head-dim elements (pairs 4c..4c+3 of the row), given the
// reciprocal rms of the whole row.  Rounding points follow the bf16 torch sequence:
// bf16(x * rrms) -> bf16(. * w) -> fp32 rotate -> bf16.
// Eight consecutive elements of one head: RMSNorm (weights wv, eight bf16) then RoPE (t0, t1 =
// cos/sin of the four pairs), operands already in registers.
__device__ __forceinline__ u32x4 norm_rope_regs(u32x4 raw, bool has_norm, float rrms, u32x4 wv, bool has_rope,
                                                f32x4 t0, f32x4 t1) {
  float v[8];
  v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x); v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
  v[4] = bf16_lo(raw.z); v[5] = bf16_hi(raw.z); v[6] = bf16_lo(raw.w); v[7] = bf16_hi(raw.w);
  if (has_norm) {
    float wf[8] = {bf16_lo(wv.x), bf16_hi(wv.x), bf16_lo(wv.y), bf16_hi(wv.y),
                   bf16_lo(wv.z), bf16_hi(wv.z), bf16_lo(wv.w), bf16_hi(wv.w)};
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = round_bf16(round_bf16(v[i] * rrms) * wf[i]);
  }
  if (has_rope) {
    float cs[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float c = cs[2 * i], s = cs[2 * i + 1];
      float x0 = v[2 * i], x1 = v[2 * i + 1];
      // same expression order as freqs[...,0]*x0 + freqs[...,1]*x1 with rows (c,-s) and (s,c)
      // (separately rounded products and sum, as separate torch ops produce them)
      v[2 * i] = mul_add_unfused(c, x0, -s, x1);
      v[2 * i + 1] = mul_add_unfused(s, x0, c, x1);
    }
  }
  u32x4 o;
  o.x = pack_bf16x2(v[0], v[1]);
  o.y = pack_bf16x2(v[2], v[3]);
  o.z = pack_bf16x2(v[4], v[5]);
  o.w = pack_bf16x2(v[6], v[7]);
  return o;
}

__device__ __forceinline__ u32x4 norm_rope_chunk(u32x4 raw, bool has_norm, float rrms,
                                                 const uint16_t* __restrict__ w8,
                                                 const float* __restrict__ cs8) {
  const u32x4 wv = has_norm ? *reinterpret_cast<const u32x4*>(w8) : u32x4{0, 0, 0, 0};
  f32x4 t0 = {0.f, 0.f, 0.f, 0.f}, t1 = t0;
  if (cs8) {
    t0 = *reinterpret_cast<const f32x4*>(cs8);
    t1 = *reinterpret_cast<const f32x4*>(cs8 + 4);
  }
  return norm_rope_regs(raw, has_norm, rrms, wv, cs8 != nullptr, t0, t1);
}

__device__ __forceinline__ float sumsq_chunk(u32x4 raw) {
  float s = 0.f;
  float a;
  a = bf16_lo(raw.x); s += a * a; a = bf16_hi(raw.x); s += a * a;
  a = bf16_lo(raw.y); s += a * a; a = bf16_hi(raw.y); s += a * a;
  a = bf16_lo(raw.z); s += a * a; a = bf16_hi(raw.z); s += a * a;
  a = bf16_lo(raw.w); s += a * a; a = bf16_hi(raw.w); s += a * a;
  return s;
}
}  // namespace dsx
#endif
