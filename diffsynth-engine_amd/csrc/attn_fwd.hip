// Flash attention forward for gfx950, head dim 128, bf16 operands, fp32 online softmax.
//
// Work split: one workgroup = 4 waves = 256 consecutive query rows of one (batch, head);
// every wave owns 64 queries (two 32-wide MFMA column tiles) and walks all keys in blocks of 64.
//
// MFMA formulation (v_mfma_f32_32x32x16_bf16, D[i][j] += sum_k A[i][k] * B[k][j]; lane (g,i)
// feeds A[i][8g..8g+7], lane (g,j) feeds B[8g..8g+7][j]; result lane (g,j) register r holds
// row 8*(r/4) + 4g + (r%4), column j):
//   S^T = K * Q^T      A = K tile (from LDS), B = Q^T (registers, loaded once)
//   O^T += V^T * P^T   A = V^T tile (from LDS), B = P^T (registers, straight from S^T)
// With the transposed formulation a lane only ever holds data of ONE query (column j), so the
// softmax row statistics are lane-local apart from one exchange between the two half-waves,
// and the S^T accumulators turn into the B operand of the second product without any shuffle:
// registers 8c..8c+7 of an S^T tile are keys {4g..4g+3, 8+4g..8+4g+3} of 16-key chunk c, and the
// V^T tile in LDS stores its key axis in exactly that slot order.
//
// LDS per stage: K tile [64 keys][128 d] (256-byte rows, 16-byte chunk c of row r stored at
// c ^ (r & 15)) and V^T tile [128 d][64 key slots] (128-byte rows, chunk c of row r stored at
// c ^ ((r/2) & 7)); both swizzles make 16 consecutive rows at one logical chunk conflict-free.
#include "attn_internal.h"
#include "common.h"

namespace dsx {

constexpr int QB = 256;   // queries per workgroup
constexpr int KB = 64;    // keys per block
constexpr int HD = 128;   // head dim
constexpr int kKTileBytes = KB * HD * 2;          // 16 KiB
constexpr int kAttnStageBytes = 2 * kKTileBytes;  // K + V^T
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ int k_lds_off(int key, int chunk) {
  return key * 256 + ((chunk ^ (key & 15)) << 4);
}
__device__ __forceinline__ int vt_lds_off(int d, int chunk) {
  return d * 128 + ((chunk ^ ((d >> 1) & 7)) << 4);
}

__device__ __forceinline__ float halfwave_allmax(float v) {
  // max over the pair of lanes (l, l^32)
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halfwave_allsum(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <bool FUSED>
__global__ __launch_bounds__(256) void attn_fwd_kernel(dsx_attn_params p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5, li = lane & 31;
  const int b = blockIdx.z, h = blockIdx.y;
  const int64_t Sq = p.sq[0] + p.sq[1];
  const int64_t Skv = p.skv[0] + p.skv[1];
  const int64_t q0 = (int64_t)blockIdx.x * QB + wave * 64;

  const uint16_t* qbase[2];
  const uint16_t* kbase[2];
  const uint16_t* vbase[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    qbase[s] = (const uint16_t*)p.q[s] + (int64_t)b * p.q_sb[s] + (int64_t)h * p.q_sh[s];
    kbase[s] = (const uint16_t*)p.k[s] + (int64_t)b * p.k_sb[s] + (int64_t)h * p.k_sh[s];
    vbase[s] = (const uint16_t*)p.v[s] + (int64_t)b * p.v_sb[s] + (int64_t)h * p.v_sh[s];
  }
  const float* rope = FUSED && p.rope ? p.rope + (int64_t)b * p.rope_sb : nullptr;

  // ---------------- Q fragments (B operand of S^T = K Q^T), loaded once ----------------
  bf16x8 qf[2][8];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    int64_t row = q0 + qt * 32 + li;
    if (row >= Sq) row = Sq - 1;
    const int seg = row >= p.sq[0] ? 1 : 0;
    const uint16_t* src = qbase[seg] + (row - (seg ? p.sq[0] : 0)) * p.q_ss[seg];
    u32x4 raw[8];
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) raw[kc] = *reinterpret_cast<const u32x4*>(src + kc * 16 + g * 8);
    if (FUSED) {
      const uint16_t* nw = (const uint16_t*)p.q_norm_w[seg];
      float rrms = 1.f;
      if (nw) {
        float ss = 0.f;
#pragma unroll
        for (int kc = 0; kc < 8; ++kc) ss += sumsq_chunk(raw[kc]);
        ss = halfwave_allsum(ss);
        rrms = rsqrtf(ss * (1.0f / HD) + p.norm_eps);
      }
#pragma unroll
      for (int kc = 0; kc < 8; ++kc)
        raw[kc] = norm_rope_chunk(raw[kc], nw != nullptr, rrms, nw ? nw + kc * 16 + g * 8 : nullptr,
                                  rope ? rope + row * HD + kc * 16 + g * 8 : nullptr);
    }
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) qf[qt][kc] = __builtin_bit_cast(bf16x8, raw[kc]);
  }

  // ---------------- K / V staging maps ----------------
  // K: chunk id = tid + 256*i -> key = id/16, chunk = id%16 (16 lanes read one 256-byte row)
  const int ks_c = tid & 15;
  const int ks_r = tid >> 4;  // +16*i
  // V: thread owns 4 keys x 8 d: dgroup = tid%16, keygroup = tid/16
  const int vs_dg = tid & 15;
  const int vs_kg = tid >> 4;
  // destination of the transposed 8-byte pieces: 16-key chunk ch, kappa0 = 4*(kg%4) = 8a + 4gg
  const int vs_ch = vs_kg >> 2;
  const int vs_a = (vs_kg >> 1) & 1;
  const int vs_gg = vs_kg & 1;
  const int vs_chunk = vs_ch * 2 + vs_gg;

  u32x4 sk[4], sv[4];
  auto load_kv = [&](int kb) {
    const int64_t key0 = (int64_t)kb * KB;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int64_t key = key0 + ks_r + 16 * i;
      if (key >= Skv) key = Skv - 1;
      const int seg = key >= p.skv[0] ? 1 : 0;
      const int64_t lrow = key - (seg ? p.skv[0] : 0);
      u32x4 raw = *reinterpret_cast<const u32x4*>(kbase[seg] + lrow * p.k_ss[seg] + ks_c * 8);
      if (FUSED) {
        const uint16_t* nw = (const uint16_t*)p.k_norm_w[seg];
        float rrms = 1.f;
        if (nw) {
          float ss = sumsq_chunk(raw);
          // the 16 lanes tid%16 of one key hold the whole 128-wide row
          ss += dpp_f32<kDppQuadXor1>(ss);
          ss += dpp_f32<kDppQuadXor2>(ss);
          ss += dpp_f32<kDppRowRor4>(ss);
          ss += dpp_f32<kDppRowRor8>(ss);
          rrms = rsqrtf(ss * (1.0f / HD) + p.norm_eps);
        }
        raw = norm_rope_chunk(raw, nw != nullptr, rrms, nw ? nw + ks_c * 8 : nullptr,
                              rope ? rope + key * HD + ks_c * 8 : nullptr);
      }
      sk[i] = raw;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int64_t key = key0 + vs_kg * 4 + i;
      if (key >= Skv) key = Skv - 1;
      const int seg = key >= p.skv[0] ? 1 : 0;
      const int64_t lrow = key - (seg ? p.skv[0] : 0);
      sv[i] = *reinterpret_cast<const u32x4*>(vbase[seg] + lrow * p.v_ss[seg] + vs_dg * 8);
    }
  };
  auto store_kv = [&](int buf) {
    uint8_t* sK = smem + buf * kAttnStageBytes;
    uint8_t* sV = sK + kKTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<u32x4*>(sK + k_lds_off(ks_r + 16 * i, ks_c)) = sk[i];
      // 4 keys x 8 d  ->  8 d-rows x 4 keys
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w0 = sv[0][j], w1 = sv[1][j], w2 = sv[2][j], w3 = sv[3][j];
      u32x2 even, odd;
      even.x = (w0 & 0xffffu) | (w1 << 16);
      even.y = (w2 & 0xffffu) | (w3 << 16);
      odd.x = (w0 >> 16) | (w1 & 0xffff0000u);
      odd.y = (w2 >> 16) | (w3 & 0xffff0000u);
      const int d = vs_dg * 8 + 2 * j;
      *reinterpret_cast<u32x2*>(sV + vt_lds_off(d, vs_chunk) + vs_a * 8) = even;
      *reinterpret_cast<u32x2*>(sV + vt_lds_off(d + 1, vs_chunk) + vs_a * 8) = odd;
    }
  };

  f32x16 oacc[4][2];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][qt][r] = 0.f;
  float m_run[2] = {-INFINITY, -INFINITY};
  float l_run[2] = {0.f, 0.f};
  const float c = p.softmax_scale * kLog2e;

  const int nkb = (int)((Skv + KB - 1) / KB);
  load_kv(0);
  store_kv(0);
  __syncthreads();

  for (int kb = 0; kb < nkb; ++kb) {
    const int buf = kb & 1;
    if (kb + 1 < nkb) load_kv(kb + 1);
    const uint8_t* sK = smem + buf * kAttnStageBytes;
    const uint8_t* sV = sK + kKTileBytes;

    // ---- S^T = K Q^T
    f32x16 s[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[kt][qt][r] = 0.f;
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        bf16x8 kf = *reinterpret_cast<const bf16x8*>(sK + k_lds_off(kt * 32 + li, 2 * kc + g));
#pragma unroll
        for (int qt = 0; qt < 2; ++qt)
          s[kt][qt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qt][kc], s[kt][qt], 0, 0, 0);
      }
    }
    // ---- mask the ragged tail of the key axis
    if ((int64_t)(kb + 1) * KB > Skv) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t key = (int64_t)kb * KB + kt * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
          if (key >= Skv) {
            s[kt][0][r] = -INFINITY;
            s[kt][1][r] = -INFINITY;
          }
        }
    }
    // ---- online softmax, one query per lane pair (l, l^32)
    bf16x8 pf[2][2][2];  // [kt][chunk][qt]
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      float mx = s[0][qt][0];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kt][qt][r]);
      mx = halfwave_allmax(mx);
      const float m_new = fmaxf(m_run[qt], mx);
      const float alpha = __builtin_amdgcn_exp2f((m_run[qt] - m_new) * c);
      const float mc = m_new * c;
      m_run[qt] = m_new;
      float lsum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        float pv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          pv[r] = __builtin_amdgcn_exp2f(s[kt][qt][r] * c - mc);
          lsum += pv[r];
        }
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
          u32x4 w;
          w.x = pack_bf16x2(pv[8 * ch + 0], pv[8 * ch + 1]);
          w.y = pack_bf16x2(pv[8 * ch + 2], pv[8 * ch + 3]);
          w.z = pack_bf16x2(pv[8 * ch + 4], pv[8 * ch + 5]);
          w.w = pack_bf16x2(pv[8 * ch + 6], pv[8 * ch + 7]);
          pf[kt][ch][qt] = __builtin_bit_cast(bf16x8, w);
        }
      }
      l_run[qt] = l_run[qt] * alpha + lsum;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[dt][qt][r] *= alpha;
      }
    }
    // ---- O^T += V^T P^T
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int ch = 0; ch < 2; ++ch)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          bf16x8 vf =
              *reinterpret_cast<const bf16x8*>(sV + vt_lds_off(dt * 32 + li, (kt * 2 + ch) * 2 + g));
#pragma unroll
          for (int qt = 0; qt < 2; ++qt)
            oacc[dt][qt] =
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kt][ch][qt], oacc[dt][qt], 0, 0, 0);
        }

    if (kb + 1 < nkb) store_kv(buf ^ 1);
    __syncthreads();
  }

  // ---------------- normalise and store.  lane (g, j): query j, d = dt*32 + 8*(r/4) + 4g + r%4
  uint16_t* obase[2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
    obase[s] = (uint16_t*)p.o[s] + (int64_t)b * p.o_sb[s] + (int64_t)h * p.o_sh[s];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    const float l = halfwave_allsum(l_run[qt]);
    const float inv = 1.0f / l;
    const int64_t row = q0 + qt * 32 + li;
    if (row < Sq) {
      const int seg = row >= p.sq[0] ? 1 : 0;
      uint16_t* dst = obase[seg] + (row - (seg ? p.sq[0] : 0)) * p.o_ss[seg];
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          u32x2 w;
          w.x = pack_bf16x2(oacc[dt][qt][4 * rq + 0] * inv, oacc[dt][qt][4 * rq + 1] * inv);
          w.y = pack_bf16x2(oacc[dt][qt][4 * rq + 2] * inv, oacc[dt][qt][4 * rq + 3] * inv);
          *reinterpret_cast<u32x2*>(dst + dt * 32 + 8 * rq + 4 * g) = w;
        }
    }
  }
}

// Standalone RMSNorm + RoPE: 16 lanes per (b,h,s) row, 16 rows per workgroup.  `out` may alias `x`
// (in-place): every thread reads its 16 bytes before it writes them.
__global__ __launch_bounds__(256) void rmsnorm_rope_kernel(
    const uint16_t* x, int64_t x_sb, int64_t x_sh, int64_t x_ss,
    const uint16_t* __restrict__ norm_w, float eps, const float* __restrict__ rope, int64_t rope_sb,
    int64_t rope_pos0, uint16_t* out, int64_t o_sb, int64_t o_sh, int64_t o_ss,
    int heads, int64_t seq) {
  const int c = threadIdx.x & 15;
  const int64_t s = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int h = blockIdx.y, b = blockIdx.z;
  const bool ok = s < seq;
  const int64_t sr = ok ? s : seq - 1;
  u32x4 raw = *reinterpret_cast<const u32x4*>(x + b * x_sb + h * x_sh + sr * x_ss + c * 8);
  float rrms = 1.f;
  if (norm_w) {
    float ss = sumsq_chunk(raw);  // 16 lanes own a row: sum within the DPP row
    ss += dpp_f32<kDppQuadXor1>(ss);
    ss += dpp_f32<kDppQuadXor2>(ss);
    ss += dpp_f32<kDppRowRor4>(ss);
    ss += dpp_f32<kDppRowRor8>(ss);
    rrms = rsqrtf(ss * (1.0f / HD) + eps);
  }
  u32x4 o = norm_rope_chunk(raw, norm_w != nullptr, rrms, norm_w ? norm_w + c * 8 : nullptr,
                            rope ? rope + b * rope_sb + (rope_pos0 + sr) * HD + c * 8 : nullptr);
  if (ok) *reinterpret_cast<u32x4*>(out + b * o_sb + h * o_sh + s * o_ss + c * 8) = o;
}


// RMSNorm + RoPE of q heads followed by k heads of one token per wavefront (head h of the token at
// x + h*x_sh; a packed qkv projection has x_sh = 128), written to `out` with its own strides (`out` may
// be `x`: in place).  Sixteen lanes own a head (16 bytes each), so one wave instruction covers four
// heads; the token's RoPE row and the two norm weights are fetched once and reused for every head.
__global__ __launch_bounds__(256) void rmsnorm_rope_qk_kernel(
    const uint16_t* x, int64_t x_sb, int64_t x_sh, int64_t x_ss, int heads_q, int heads_k,
    const uint16_t* __restrict__ wq, const uint16_t* __restrict__ wk, float eps,
    const float* __restrict__ rope, int64_t rope_sb, int64_t rope_pos0, int64_t seq,
    uint16_t* out, int64_t o_sb, int64_t o_sh, int64_t o_ss) {
  const int lane = threadIdx.x & 63;
  const int c = lane & 15, hq = lane >> 4;
  const int64_t s = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int b = blockIdx.y;
  if (s >= seq) return;  // whole wavefront
  const uint16_t* row = x + b * x_sb + s * x_ss + c * 8;
  uint16_t* orow = out + b * o_sb + s * o_ss + c * 8;
  const float* cs = rope ? rope + b * rope_sb + (rope_pos0 + s) * HD + c * 8 : nullptr;
  const int total = heads_q + heads_k;
  const u32x4 zero4 = {0, 0, 0, 0};
  const u32x4 wvq = wq ? *reinterpret_cast<const u32x4*>(wq + c * 8) : zero4;
  const u32x4 wvk = wk ? *reinterpret_cast<const u32x4*>(wk + c * 8) : zero4;
  f32x4 t0 = {0.f, 0.f, 0.f, 0.f}, t1 = t0;
  if (cs) {
    t0 = *reinterpret_cast<const f32x4*>(cs);
    t1 = *reinterpret_cast<const f32x4*>(cs + 4);
  }
  for (int h0 = 0; h0 < total; h0 += 16) {
    u32x4 raw[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = min(h0 + i * 4 + hq, total - 1);
      raw[i] = *reinterpret_cast<const u32x4*>(row + h * x_sh);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = h0 + i * 4 + hq;
      const uint16_t* w = h < heads_q ? wq : wk;
      float rrms = 1.f;
      if (w) {
        float ss = sumsq_chunk(raw[i]);
        ss += dpp_f32<kDppQuadXor1>(ss);
        ss += dpp_f32<kDppQuadXor2>(ss);
        ss += dpp_f32<kDppRowRor4>(ss);
        ss += dpp_f32<kDppRowRor8>(ss);
        rrms = rsqrtf(ss * (1.0f / HD) + eps);
      }
      const u32x4 o = norm_rope_regs(raw[i], w != nullptr, rrms, h < heads_q ? wvq : wvk, cs != nullptr, t0, t1);
      if (h < total) *reinterpret_cast<u32x4*>(orow + h * o_sh) = o;
    }
  }
}

}  // namespace dsx

static int check_seg(const void* const* ptr, const int64_t* len) {
  for (int g = 0; g < 2; ++g) {
    if (len[g] < 0) return DSX_EBADSHAPE;
    if (len[g] > 0 && !ptr[g]) return DSX_ENULL;
    if (((uintptr_t)ptr[g]) & 15) return DSX_EALIGN;
  }
  return DSX_OK;
}

extern "C" int dsx_attn_fwd(const dsx_attn_params* p, void* stream) {
  using namespace dsx;
  if (!p) return DSX_ENULL;
  if (p->head_dim != HD || p->batch <= 0 || p->heads <= 0) return DSX_EBADSHAPE;
  if (p->batch > 65535 || p->heads > 65535) return DSX_EBADSHAPE;
  int rc;
  if ((rc = check_seg(p->q, p->sq)) || (rc = check_seg(p->k, p->skv)) ||
      (rc = check_seg(p->v, p->skv)) || (rc = check_seg((const void* const*)p->o, p->sq)))
    return rc;
  const int64_t Sq = p->sq[0] + p->sq[1], Skv = p->skv[0] + p->skv[1];
  if (Sq <= 0 || Skv <= 0 || Sq > (1ll << 30) || Skv > (1ll << 30)) return DSX_EBADSHAPE;
  for (int g = 0; g < 2; ++g) {
    const int64_t strides[12] = {p->q_sb[g], p->q_sh[g], p->q_ss[g], p->k_sb[g], p->k_sh[g], p->k_ss[g],
                                 p->v_sb[g], p->v_sh[g], p->v_ss[g], p->o_sb[g], p->o_sh[g], p->o_ss[g]};
    for (int i = 0; i < 12; ++i)
      if (strides[i] & 7) return DSX_EALIGN;  // every row start must stay 16-byte aligned
    if (p->sq[g] > 1 && (p->o_ss[g] < HD || p->q_ss[g] < HD)) return DSX_EBADSHAPE;
  }
  const bool fused = p->rope || p->q_norm_w[0] || p->q_norm_w[1] || p->k_norm_w[0] || p->k_norm_w[1];
  if (p->rope && (((uintptr_t)p->rope & 15) || (p->rope_sb & 3))) return DSX_EALIGN;
  if (p->rope && Sq != Skv) return DSX_EBADSHAPE;  // fused RoPE is defined for self/joint attention
  for (int g = 0; g < 2; ++g)
    if (((uintptr_t)p->q_norm_w[g] & 15) || ((uintptr_t)p->k_norm_w[g] & 15)) return DSX_EALIGN;

  if (p->workspace && ((uintptr_t)p->workspace & 15)) return DSX_EALIGN;
  if (!fused) return launch_attn_plain(*p, p->workspace, p->workspace ? p->workspace_bytes : 0, (hipStream_t)stream);

  // With caller scratch: k is normalised / rotated ONCE into it by a row kernel (every query block of a
  // head reads all of k), while q gets the same treatment for free inside the attention kernel, where each
  // row is read exactly once.
  const bool k_side = p->rope || p->k_norm_w[0] || p->k_norm_w[1];
  if (!k_side) return launch_attn_plain(*p, nullptr, 0, (hipStream_t)stream);  // q only: nothing to copy
  const int64_t ws_need = 2 * (int64_t)p->batch * p->heads * Skv * HD;
  if (p->workspace && p->workspace_bytes >= ws_need) {
    hipStream_t st = (hipStream_t)stream;
    dsx_attn_params t = *p;
    uint16_t* base = (uint16_t*)p->workspace;
    const int64_t o_sh = Skv * HD, o_sb = (int64_t)p->heads * Skv * HD;  // the copy is (batch, head, key, 128)
    int64_t row0 = 0;
    for (int g = 0; g < 2; ++g) {
      const int64_t n = p->skv[g];
      uint16_t* dst = base + row0 * HD;
      if (n > 0) {
        // 16 lanes per (token, head) row.  (The wavefront-per-token kernel of dsx_rmsnorm_rope_qk was
        // measured here too, with a head-major and with a token-major copy: 16.2 us against 15.1 us.)
        dim3 grid((unsigned)((n + 15) / 16), (unsigned)p->heads, (unsigned)p->batch), block(256);
        rmsnorm_rope_kernel<<<grid, block, 0, st>>>((const uint16_t*)p->k[g], p->k_sb[g], p->k_sh[g], p->k_ss[g],
                                                    (const uint16_t*)p->k_norm_w[g], p->norm_eps, p->rope,
                                                    p->rope_sb, row0, dst, o_sb, o_sh, HD, p->heads, n);
      }
      t.k[g] = n > 0 ? dst : nullptr;
      t.k_sb[g] = o_sb;
      t.k_sh[g] = o_sh;
      t.k_ss[g] = HD;
      row0 += n;
    }
    if (hipGetLastError() != hipSuccess) return DSX_ELAUNCH;
    t.k_norm_w[0] = t.k_norm_w[1] = nullptr;  // q_norm_w and rope stay: the attention kernel applies them to q
    return launch_attn_plain(t, nullptr, 0, st);
  }

  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)attn_fwd_kernel<false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            2 * kAttnStageBytes) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_fwd_kernel<true>,
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            2 * kAttnStageBytes) != hipSuccess)
      return DSX_ELAUNCH;
    attr_set = true;
  }
  dim3 grid((unsigned)((Sq + QB - 1) / QB), (unsigned)p->heads, (unsigned)p->batch), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (fused)
    attn_fwd_kernel<true><<<grid, block, 2 * kAttnStageBytes, st>>>(*p);
  else
    attn_fwd_kernel<false><<<grid, block, 2 * kAttnStageBytes, st>>>(*p);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

extern "C" int dsx_rmsnorm_rope(const void* x, int64_t x_sb, int64_t x_sh, int64_t x_ss,
                                const void* norm_w, float eps, const float* rope, int64_t rope_sb,
                                int64_t rope_pos0, void* out, int64_t o_sb, int64_t o_sh,
                                int64_t o_ss, int32_t batch, int32_t heads, int64_t seq,
                                void* stream) {
  using namespace dsx;
  if (!x || !out) return DSX_ENULL;
  if (batch <= 0 || heads <= 0 || seq < 0 || batch > 65535 || heads > 65535) return DSX_EBADSHAPE;
  if ((x_sb | x_sh | x_ss | o_sb | o_sh | o_ss) & 7) return DSX_EALIGN;
  if (((uintptr_t)x & 15) || ((uintptr_t)out & 15) || ((uintptr_t)norm_w & 15) ||
      ((uintptr_t)rope & 15) || (rope_sb & 3))
    return DSX_EALIGN;
  if (seq == 0) return DSX_OK;
  dim3 grid((unsigned)((seq + 15) / 16), (unsigned)heads, (unsigned)batch), block(256);
  rmsnorm_rope_kernel<<<grid, block, 0, (hipStream_t)stream>>>(
      (const uint16_t*)x, x_sb, x_sh, x_ss, (const uint16_t*)norm_w, eps, rope, rope_sb, rope_pos0,
      (uint16_t*)out, o_sb, o_sh, o_ss, heads, seq);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

extern "C" int dsx_rmsnorm_rope_qk(void* x, int64_t x_sb, int64_t x_ss, int32_t heads_q, int32_t heads_k,
                                   const void* q_norm_w, const void* k_norm_w, float eps, const float* rope,
                                   int64_t rope_sb, int64_t rope_pos0, int32_t batch, int64_t seq,
                                   void* stream) {
  using namespace dsx;
  if (!x) return DSX_ENULL;
  if (batch <= 0 || heads_q < 0 || heads_k < 0 || heads_q + heads_k <= 0 || heads_q + heads_k > 65535 ||
      seq < 0 || batch > 65535)
    return DSX_EBADSHAPE;
  if (seq > 1 && x_ss < (int64_t)(heads_q + heads_k) * HD) return DSX_EBADSHAPE;
  if ((x_sb | x_ss) & 7) return DSX_EALIGN;
  if (((uintptr_t)x & 15) || ((uintptr_t)q_norm_w & 15) || ((uintptr_t)k_norm_w & 15) ||
      ((uintptr_t)rope & 15) || (rope_sb & 3))
    return DSX_EALIGN;
  if (seq == 0) return DSX_OK;
  dim3 grid((unsigned)((seq + 3) / 4), (unsigned)batch), block(256);
  rmsnorm_rope_qk_kernel<<<grid, block, 0, (hipStream_t)stream>>>(
      (const uint16_t*)x, x_sb, HD, x_ss, heads_q, heads_k, (const uint16_t*)q_norm_w, (const uint16_t*)k_norm_w,
      eps, rope, rope_sb, rope_pos0, seq, (uint16_t*)x, x_sb, HD, x_ss);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

extern "C" int64_t dsx_attn_workspace_bytes(const dsx_attn_params* p) {
  using namespace dsx;
  if (!p || p->head_dim != HD || p->batch <= 0 || p->heads <= 0) return 0;
  const int64_t Sq = p->sq[0] + p->sq[1], Skv = p->skv[0] + p->skv[1];
  if (Sq <= 0 || Skv <= 0 || Sq > (1ll << 30) || Skv > (1ll << 30)) return 0;
  const bool k_side = p->rope || p->k_norm_w[0] || p->k_norm_w[1];
  const int64_t copies = k_side ? 2 * (int64_t)p->batch * p->heads * Skv * HD : 0;
  return copies + attn_plain_workspace_bytes(*p);
}
