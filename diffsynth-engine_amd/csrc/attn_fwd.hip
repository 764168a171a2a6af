// Attention entry points of the C ABI (dsx_attn_fwd and its allocation-free twin) and the row kernels that
// apply the per-head RMSNorm and the RoPE rotation to q and k ahead of the attention kernel.
//
// RMSNorm / RoPE requested from dsx_attn_fwd are applied to q inside the attention kernel (attn_plain.hip: every
// query row is read exactly once there) and to k by ONE pass of rmsnorm_rope_kernel into scratch memory (every
// query block of a head reads all of that head's k, so per-block recomputation would repeat the work 18 times at
// 4608 tokens).  The scratch is the caller's (dsx_attn_fwd) or a static device array (dsx_attn_fwd_static).
#include "attn_internal.h"
#include "common.h"

namespace dsx {

constexpr int HD = 128;   // head dim

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

// Everything dsx_attn_fwd refuses before a kernel is launched: shapes, strides, alignment, the extent of the
// RoPE table.  The kernels index with these values unchecked.
static int attn_validate(const dsx_attn_params* p) {
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
    // rows of one head must not overlap: a row is 128 elements
    if (p->sq[g] > 1 && (p->o_ss[g] < HD || p->q_ss[g] < HD)) return DSX_EBADSHAPE;
    if (p->skv[g] > 1 && (p->k_ss[g] < HD || p->v_ss[g] < HD)) return DSX_EBADSHAPE;
  }
  if (p->rope) {
    if (((uintptr_t)p->rope & 15) || (p->rope_sb & 3)) return DSX_EALIGN;
    if (Sq != Skv) return DSX_EBADSHAPE;        // fused RoPE is defined for self/joint attention
    if (p->rope_rows < Sq) return DSX_EBADSHAPE;  // the table must hold a row for every joint position
    if (p->batch > 1 && p->rope_sb != 0 && p->rope_sb < p->rope_rows * HD) return DSX_EBADSHAPE;
  }
  for (int g = 0; g < 2; ++g)
    if (((uintptr_t)p->q_norm_w[g] & 15) || ((uintptr_t)p->k_norm_w[g] & 15)) return DSX_EALIGN;
  if (p->workspace && ((uintptr_t)p->workspace & 15)) return DSX_EALIGN;
  if (p->workspace && p->workspace_bytes < 0) return DSX_EBADSHAPE;
  if (p->qk_norm2_max) {
    if ((uintptr_t)p->qk_norm2_max & 3) return DSX_EALIGN;
    // the two maxima describe q and k as given; fused pre-processing would change the rows behind them
    if (p->rope || p->q_norm_w[0] || p->q_norm_w[1] || p->k_norm_w[0] || p->k_norm_w[1]) return DSX_EBADSHAPE;
  }
  return DSX_OK;
}

static int64_t attn_k_copy_bytes(const dsx_attn_params* p) {
  const bool k_side = p->rope || p->k_norm_w[0] || p->k_norm_w[1];
  return k_side ? 2 * (int64_t)p->batch * p->heads * (p->skv[0] + p->skv[1]) * dsx::HD : 0;
}

// The launches of one validated call, with `ws` (ws_bytes) as its scratch; allocates nothing.
static int attn_run(const dsx_attn_params* p, void* ws, int64_t ws_bytes, hipStream_t st) {
  using namespace dsx;
  const int64_t Skv = p->skv[0] + p->skv[1];
  const int64_t copy_bytes = attn_k_copy_bytes(p);
  if (copy_bytes == 0)  // plain, or q-side pre-processing only: nothing to copy, the scratch serves the key split
    return launch_attn_plain(*p, ws, ws ? ws_bytes : 0, st);
  // k is normalised / rotated ONCE into the scratch by a row kernel (every query block of a head reads all of
  // k), while q gets the same treatment for free inside the attention kernel, where each row is read once.
  if (!ws || ws_bytes < copy_bytes) return DSX_EWORKSPACE;
  dsx_attn_params t = *p;
  uint16_t* base = (uint16_t*)ws;
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

extern "C" int dsx_attn_fwd(const dsx_attn_params* p, void* stream) {
  const int rc = attn_validate(p);
  if (rc != DSX_OK) return rc;
  return attn_run(p, p->workspace, p->workspace ? p->workspace_bytes : 0, (hipStream_t)stream);
}

extern "C" int64_t dsx_attn_workspace_bytes(const dsx_attn_params* p) {
  using namespace dsx;
  if (!p || p->head_dim != HD || p->batch <= 0 || p->heads <= 0) return 0;
  const int64_t Sq = p->sq[0] + p->sq[1], Skv = p->skv[0] + p->skv[1];
  if (Sq <= 0 || Skv <= 0 || Sq > (1ll << 30) || Skv > (1ll << 30)) return 0;
  // A call that copies k launches the attention kernel without scratch of its own (attn_run), so the copy is all
  // it needs; only a call without a copy can use scratch for the key-range split.
  const int64_t copy_bytes = attn_k_copy_bytes(p);
  return copy_bytes > 0 ? copy_bytes : attn_plain_workspace_bytes(*p);
}

// ---- the allocation-free twin: the same launches over a static device array ------------------------------
// Every GPU the library runs on holds its own copy of the array at its own address; the host-side name is only
// a handle for hipGetSymbolAddress, never a pointer a kernel could use.
namespace {
__device__ __align__(256) unsigned char scratch[DSX_ATTN_STATIC_SCRATCH_BYTES];
dsx::PerDeviceOnce g_scratch_once;
void* g_scratch_ptr[dsx::kMaxDevices];  // per device, resolved on the first call made with that device current
}  // namespace

// Device address of the current device's copy of `scratch` (resolved once per device, under a lock).
static int attn_static_scratch(void** out) {
  const int rc = dsx::per_device_once(g_scratch_once, [](int dev) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return (int)DSX_ELAUNCH;
    g_scratch_ptr[dev] = ptr;
    return (int)DSX_OK;
  });
  if (rc != DSX_OK) return rc;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= dsx::kMaxDevices) return DSX_EARCH;
  *out = g_scratch_ptr[dev];
  return DSX_OK;
}

extern "C" int64_t dsx_attn_static_scratch_bytes(void) { return DSX_ATTN_STATIC_SCRATCH_BYTES; }

extern "C" int dsx_attn_fwd_static(const dsx_attn_params* p, void* stream) {
  int rc = attn_validate(p);
  if (rc != DSX_OK) return rc;
  if (p->workspace) return DSX_EBADSHAPE;  // this entry point owns its scratch; a caller's buffer goes to dsx_attn_fwd
  const int64_t need = dsx_attn_workspace_bytes(p);
  if (need > DSX_ATTN_STATIC_SCRATCH_BYTES) return DSX_EWORKSPACE;
  void* ws = nullptr;
  if (need > 0 && (rc = attn_static_scratch(&ws)) != DSX_OK) return rc;
  return attn_run(p, ws, need > 0 ? DSX_ATTN_STATIC_SCRATCH_BYTES : 0, (hipStream_t)stream);
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
