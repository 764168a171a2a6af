// FP8 e4m3 scaled GEMM for gfx950:  out = bf16((A * W^T) * a_scale[m] * w_scale + bias[n]).
//
// Both operands are K-contiguous, which is what v_mfma_f32_16x16x128_f8f6f4 wants: lane
// (q = lane/16, i = lane%16) feeds 32 K-bytes of row i of the first operand and of column i of
// the second.  Any permutation of K applied to both operands leaves the product unchanged, so
// the loaders only have to keep the two consistent.
// (On random e4m3 operands, where the chip runs at its power limit, a bare stream of this shape sustains 9 % more
// than one of v_mfma_f32_32x32x64_f8f6f4 -- 4.13 against 3.79 PFLOP/s -- while both reach the 5.0 PFLOP/s peak on
// all-zero operands; the generic kernel for odd shapes below still uses the larger shape.)
//
// The kernels compute C^T tiles (first operand = W rows, second = A rows): the accumulator of
// lane (q, i) then holds ONE token m = i and four consecutive output features, so the per-token
// scale is a per-lane constant and the bf16 results leave as 8-byte pieces.
//
// Main kernel: 256x256 output tile per workgroup, 8 waves as 2x4, each wave 128 (n) x 64 (m) = 8x4 MFMA
// tiles (128 fp32 accumulators), two waves per SIMD.  Operands reach LDS by global_load_lds_dwordx4
// (HBM/L2 -> LDS without staging registers) in 128-byte-wide units through a five-slot ring; MFMA
// operand fragments are read ahead of their use so that LDS reads overlap the MFMAs.  LDS rows are
// 128 B (8 chunks of 16 B); chunk c of row r lives at chunk c ^ ((r/2)&7), which makes 16 lanes
// reading 16 consecutive rows at one logical chunk hit 16 distinct bank groups.
// One launch can carry two independent problems (the image- and text-stream linears of a joint
// block): their tiles share the grid, so the small problem runs on CUs the large one leaves idle.
// A launch with at most 128 such tiles (half the compute units) runs the same kernel with four waves as
// 2x2 on tiles of 256 (n) x 128 (m) instead: twice as many workgroups, same wave tile, same K order,
// same bits.
#include "attn_internal.h"
#include "common.h"

namespace dsx {

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kTileBytes = 256 * BK;           // one operand tile, 32 KiB
constexpr int kStageBytes = 2 * kTileBytes;    // W tile + A tile, 64 KiB

__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * BK + ((chunk ^ ((row >> 1) & 7)) << 4);
}

struct GemmArgs {
  const uint8_t* a;
  const uint8_t* w;
  const float* a_scale;
  const float* w_scale;
  const uint16_t* bias;
  uint16_t* out;
  int64_t lda, ldw, ldo;
  int M, N, K;
  int tiles_m, tiles_n;
  // optional fused gated residual: out = resid + gate * bf16(acc*scale + bias)
  const uint16_t* resid;
  const uint16_t* gate;  // (N,) per batch entry, batch = row / rows_per_batch; NULL = gate of 1
  int64_t ldr, gate_sb;
  int rows_per_batch;
  // optional per-output-row weight scale (GEMV path only)
  const float* w_row_scale;
  // optional RMSNorm + RoPE of the q and k heads of a packed qkv projection, applied to the bf16 result before
  // it is stored (main kernel only): columns [0, 128*qk_heads) are q heads, the next 128*qk_heads are k heads
  const uint16_t* qk_wq;  // (128,) bf16 or NULL
  const uint16_t* qk_wk;
  const float* rope;      // (rows, 64, 2) fp32 (cos, sin) or NULL; row = rope_pos0 + m % rows_per_batch
  int64_t rope_sb;        // per batch entry m / rows_per_batch
  int rope_pos0, qk_heads;
  float qk_eps;
  // optional second segment of the reduction axis (main kernel only): K2 more columns from (a2, w2)
  const uint8_t* a2;
  const uint8_t* w2;
  int64_t lda2, ldw2;
  int K2;
};

// Two problems in one grid: logical tiles [0, tiles of p[0]) belong to p[0], the rest to p[1].
struct GemmPair {
  GemmArgs p[2];
  int total0;  // tiles of p[0]
  int total;   // tiles of both
};

// Field-wise select (all operands are wave-uniform, so this is a run of scalar selects; indexing
// the kernel argument dynamically would copy both structs to scratch memory).
__device__ __forceinline__ GemmArgs pick(const GemmPair& q, bool second) {
  GemmArgs r;
#define DSX_PICK(f) r.f = second ? q.p[1].f : q.p[0].f
  DSX_PICK(a); DSX_PICK(w); DSX_PICK(a_scale); DSX_PICK(w_scale); DSX_PICK(bias); DSX_PICK(out);
  DSX_PICK(lda); DSX_PICK(ldw); DSX_PICK(ldo); DSX_PICK(M); DSX_PICK(N); DSX_PICK(K);
  DSX_PICK(tiles_m); DSX_PICK(tiles_n); DSX_PICK(resid); DSX_PICK(gate); DSX_PICK(ldr); DSX_PICK(gate_sb);
  DSX_PICK(rows_per_batch); DSX_PICK(w_row_scale);
  DSX_PICK(qk_wq); DSX_PICK(qk_wk); DSX_PICK(rope); DSX_PICK(rope_sb); DSX_PICK(rope_pos0); DSX_PICK(qk_heads);
  DSX_PICK(qk_eps); DSX_PICK(a2); DSX_PICK(w2); DSX_PICK(lda2); DSX_PICK(ldw2); DSX_PICK(K2);
#undef DSX_PICK
  return r;
}

// Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of logical tile
// ids so that tiles sharing A rows / W rows meet in the same L2.
__device__ __forceinline__ int logical_tile(int wg, int total) {
  const int per_xcd = (total + 7) >> 3;
  return (wg & 7) * per_xcd + (wg >> 3);
}

__device__ __forceinline__ void tile_of(int L, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int G = 4;
  const int span = G * tiles_n;
  const int group = L / span;
  const int first_m = group * G;
  const int gsz = min(tiles_m - first_m, G);
  const int rem = L - group * span;
  tm = first_m + rem % gsz;
  tn = rem / gsz;
}

__device__ __forceinline__ void tile_coords(int wg, int tiles_m, int tiles_n, int& tm, int& tn,
                                            bool& valid) {
  const int total = tiles_m * tiles_n;
  const int L = logical_tile(wg, total);
  valid = L < total;
  tile_of(L, tiles_m, tiles_n, tm, tn);
}

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// resid + bf16(gate * proj) for one element; proj is already rounded to bf16.
__device__ __forceinline__ float residual_combine(const GemmArgs& p, float proj, int m, int n) {
  const float rv = bf16_bits_to_f32(p.resid[(int64_t)m * p.ldr + n]);
  if (p.gate)
    proj = round_bf16(bf16_bits_to_f32(p.gate[(int64_t)(m / p.rows_per_batch) * p.gate_sb + n]) * proj);
  return rv + proj;
}

// Store one C^T accumulator tile set of a wave.  acc[tn][tm]: rows n, columns m (see header).
__device__ __forceinline__ void store_ct(const GemmArgs& p, f32x16 (&acc)[4][4], int n_base,
                                         int m_base, int g, int li) {
  const float ws = p.w_scale ? *p.w_scale : 1.0f;
  const bool vec_ok = ((p.ldo & 3) == 0) && ((p.N & 3) == 0) && (((uintptr_t)p.out & 7) == 0);
#pragma unroll
  for (int tm = 0; tm < 4; ++tm) {
    const int m = m_base + tm * 32 + li;
    if (m >= p.M) continue;
    const float sc = (p.a_scale ? p.a_scale[m] : 1.0f) * ws;
    uint16_t* orow = p.out + (int64_t)m * p.ldo;
#pragma unroll
    for (int tn = 0; tn < 4; ++tn) {
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int n = n_base + tn * 32 + 8 * rq + 4 * g;
        if (vec_ok) {
          if (n < p.N) {
            float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
            if (p.bias) {
              const u32x2 bw = *reinterpret_cast<const u32x2*>(p.bias + n);
              b0 = bf16_lo(bw.x); b1 = bf16_hi(bw.x); b2 = bf16_lo(bw.y); b3 = bf16_hi(bw.y);
            }
            u32x2 o;
            float r[4] = {acc[tn][tm][4 * rq + 0] * sc + b0, acc[tn][tm][4 * rq + 1] * sc + b1,
                          acc[tn][tm][4 * rq + 2] * sc + b2, acc[tn][tm][4 * rq + 3] * sc + b3};
            if (p.resid) {
#pragma unroll
              for (int e = 0; e < 4; ++e) r[e] = residual_combine(p, round_bf16(r[e]), m, n + e);
            }
            o.x = pack_bf16x2(r[0], r[1]);
            o.y = pack_bf16x2(r[2], r[3]);
            *reinterpret_cast<u32x2*>(orow + n) = o;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e < p.N) {
              const float bj = p.bias ? bf16_bits_to_f32(p.bias[n + e]) : 0.f;
              float r = acc[tn][tm][4 * rq + e] * sc + bj;
              if (p.resid) r = residual_combine(p, round_bf16(r), m, n + e);
              orow[n + e] = (uint16_t)f32_to_bf16_bits(r);
            }
          }
        }
      }
    }
  }
}

// LDS-staged store of a wave's 64 (m) x 128 (n) block: the C^T accumulators are scaled, biased, rounded to
// bf16 and written to a wave-private LDS region as [m][n] rows (272-byte pitch: 256 data bytes + 16 pad, so
// 8-byte column writes of 32 consecutive rows spread over the banks), then read back as 16-byte chunks
// along n so that 16 lanes emit one contiguous 256-byte row segment.
constexpr int kEpiPitch = 272;
constexpr int kMainLdsBytes = 160 * 1024;  // five operand stages; the epilogue staging (136 KiB) reuses them

constexpr int SK = 64;                   // K bytes per MFMA step
constexpr int UK = 128;                  // K bytes per unit row
constexpr int NSLOT = 5;
constexpr int kUnitBytes = 256 * UK;     // 32 KiB

// 128-byte rows: 16-byte chunk c of row r lives at chunk c ^ ((r/2)&7); two rows span the 64 banks.
__device__ __forceinline__ int unit_off(int row, int chunk) {
  return row * UK + ((chunk ^ ((row >> 1) & 7)) << 4);
}

// ------------------------------------------------------------------------------------------
// Main kernel: K % 128 == 0.  Operands move HBM -> LDS in units of one operand x 128 bytes of K
// (256 rows x 128 B = 32 KiB), so that every async load instruction (64 lanes x 16 B) fetches
// eight whole 128-byte cache lines: with 64-byte rows each line would be requested twice, a step
// apart, and the second request stalls the L1 behind the still-pending first one.  Five unit
// slots (160 KiB) form a ring W0 A0 W1 A1 W2 | A2 W3 ...; one unit is one K extent of the MFMA.
// Eight waves as 2 (n) x 4 (m), each 128 (n) x 64 (m) = 8x4 MFMA tiles (128 accumulators), so that two
// waves share a SIMD: while one waits at the unit's barrier or for its operands, the other's MFMAs keep
// the matrix pipe busy, and the two overlap their epilogues.  (Four waves of 128 x 128, one per SIMD, read a
// third fewer fragment bytes per MFMA: with this file's kernel instantiated that way -- MT = 8 -- the plain
// product is 1-2 % faster and the residual and q/k epilogues, which a lone wave cannot overlap with anything,
// 3-10 % slower; a whole Flux step measures the same either way.)
// ------------------------------------------------------------------------------------------
constexpr int kEpiBytesPerWave = 64 * kEpiPitch;  // 17 408; eight of them fit the operand stages

template <int MT>
struct EpiOperands {
  u32x2 bias[8];  // [tn]: 4 consecutive bf16 at n = tn*16 + 4*q
  float sc[MT];   // [tm]: a_scale[m] * w_scale, m = tm*16 + i
};

// QK: the wave's 128 columns are one head of a packed qkv projection; q and k heads get the per-head RMSNorm and
// the RoPE rotation (same helper and rounding points as rmsnorm_rope_qk_kernel, so the result is bit-identical to
// that kernel run in place on the stored projection) between the LDS read-back and the global store: there the
// 16 lanes of a DPP row hold one token's whole head row, 16 bytes each.
// MT: 16-token accumulator columns of the wave (4 or 8); HB: which 64 tokens (four columns) of them this call
// stores; m_base is the first of those 64 tokens.
template <bool RESID, bool QK, int MT, int HB>
__device__ __forceinline__ void store_ct_lds(const GemmArgs& p, f32x4 (&acc)[8][MT], const EpiOperands<MT>& e,
                                              uint8_t* wave_lds, int n_base, int m_base, int lane) {
  const int q = lane >> 4, i16 = lane & 15;
  // One half (32 token rows = two accumulator columns tm) at a time: scale, add bias, round, stage in LDS.  The
  // global stores of the first half are then in flight while the second half is converted.
  auto stage_half = [&](int h) {
#pragma unroll
    for (int tmi = 0; tmi < 2; ++tmi) {
      const int tl = 2 * h + tmi, tm = HB * 4 + tl;
      const float sc = e.sc[tm];
      uint8_t* lrow = wave_lds + (tl * 16 + i16) * kEpiPitch;
#pragma unroll
      for (int tn = 0; tn < 8; ++tn) {
        const int nl = tn * 16 + 4 * q;
        const u32x2 bw = e.bias[tn];
        u32x2 o;
        o.x = pack_bf16x2(acc[tn][tm][0] * sc + bf16_lo(bw.x), acc[tn][tm][1] * sc + bf16_hi(bw.x));
        o.y = pack_bf16x2(acc[tn][tm][2] * sc + bf16_lo(bw.y), acc[tn][tm][3] * sc + bf16_hi(bw.y));
        *reinterpret_cast<u32x2*>(lrow + nl * 2) = o;
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the region is private to this wave
    __builtin_amdgcn_wave_barrier();
  };
  const int ch = lane & 15, r0 = lane >> 4;
  const int n = n_base + ch * 8;
  const bool col_ok = n < p.N;
  u32x4 gv = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  bool gate_per_row = false;
  const bool gated = RESID && p.gate != nullptr;
  if (gated) {
    const int b_lo = m_base / p.rows_per_batch, b_hi = min(m_base + 63, p.M - 1) / p.rows_per_batch;
    gate_per_row = b_lo != b_hi;
    if (!gate_per_row && col_ok) gv = *reinterpret_cast<const u32x4*>(p.gate + (int64_t)b_lo * p.gate_sb + n);
  }
  uint16_t* const out_lane = p.out + (int64_t)(m_base + r0) * p.ldo + n;
  const uint16_t* const res_lane = RESID ? p.resid + (int64_t)(m_base + r0) * p.ldr + n : nullptr;
  const int64_t out_step = 4 * p.ldo, res_step = 4 * p.ldr;
  // QK pre-processing of this wave's head (wave-uniform choices): which norm weight, whether anything applies
  const bool qk_is_q = QK && n_base < p.qk_heads * 128;
  const bool qk_on = QK && n_base < 2 * p.qk_heads * 128;
  const uint16_t* const qk_w = qk_is_q ? p.qk_wq : p.qk_wk;
  u32x4 qk_wv = {0, 0, 0, 0};
  if (QK && qk_on && qk_w) qk_wv = *reinterpret_cast<const u32x4*>(qk_w + ch * 8);
  const bool qk_one_batch = m_base + 63 < p.rows_per_batch;  // wave-uniform: no division per row
  auto rows8 = [&](int it0, bool guarded) {
    u32x4 v[8], rv[8];
    bool ok[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int ml = (it0 + u) * 4 + r0;
      const int m = m_base + ml;
      ok[u] = !guarded || (m < p.M && col_ok);
      v[u] = *reinterpret_cast<const u32x4*>(wave_lds + ml * kEpiPitch + ch * 16);
      if (RESID && ok[u]) rv[u] = *reinterpret_cast<const u32x4*>(res_lane + (it0 + u) * res_step);
    }
    if (QK && qk_on) {
      f32x4 t0[8], t1[8];
      if (p.rope) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {  // rows past M are never stored: their table address is clamped, not predicated
          const int m = min(m_base + (it0 + u) * 4 + r0, p.M - 1);
          const int b = qk_one_batch ? 0 : m / p.rows_per_batch;
          const float* cs = p.rope + (int64_t)b * p.rope_sb +
                            (int64_t)(p.rope_pos0 + m - b * p.rows_per_batch) * 128 + ch * 8;
          t0[u] = *reinterpret_cast<const f32x4*>(cs);
          t1[u] = *reinterpret_cast<const f32x4*>(cs + 4);
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        float rrms = 1.f;
        if (qk_w) {
          float ss = sumsq_chunk(v[u]);  // the 16 lanes of a DPP row hold the head row
          ss += dpp_f32<kDppQuadXor1>(ss);
          ss += dpp_f32<kDppQuadXor2>(ss);
          ss += dpp_f32<kDppRowRor4>(ss);
          ss += dpp_f32<kDppRowRor8>(ss);
          rrms = rsqrtf(ss * (1.0f / 128) + p.qk_eps);
        }
        v[u] = norm_rope_regs(v[u], qk_w != nullptr, rrms, qk_wv, p.rope != nullptr, t0[u], t1[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int m = m_base + (it0 + u) * 4 + r0;
      if (!ok[u]) continue;
      if (RESID) {
        u32x4 gu = gv;
        if (gate_per_row)
          gu = *reinterpret_cast<const u32x4*>(p.gate + (int64_t)(m / p.rows_per_batch) * p.gate_sb + n);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const float t0 = gated ? round_bf16(bf16_lo(gu[c]) * bf16_lo(v[u][c])) : bf16_lo(v[u][c]);
          const float t1 = gated ? round_bf16(bf16_hi(gu[c]) * bf16_hi(v[u][c])) : bf16_hi(v[u][c]);
          v[u][c] = pack_bf16x2(bf16_lo(rv[u][c]) + t0, bf16_hi(rv[u][c]) + t1);
        }
      }
      *reinterpret_cast<u32x4*>(out_lane + (it0 + u) * out_step) = v[u];
    }
  };
  // interior tile with a residual: each half's eight residual rows are requested before that half is
  // converted, so that their latency passes under the conversion instead of after the LDS read-back
  auto rows8_prefetched = [&](int it0, u32x4 (&rv)[8]) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      v[u] = *reinterpret_cast<const u32x4*>(wave_lds + ((it0 + u) * 4 + r0) * kEpiPitch + ch * 16);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      u32x4 gu = gv;
      if (gate_per_row)
        gu = *reinterpret_cast<const u32x4*>(
            p.gate + (int64_t)((m_base + (it0 + u) * 4 + r0) / p.rows_per_batch) * p.gate_sb + n);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float t0 = gated ? round_bf16(bf16_lo(gu[c]) * bf16_lo(v[u][c])) : bf16_lo(v[u][c]);
        const float t1 = gated ? round_bf16(bf16_hi(gu[c]) * bf16_hi(v[u][c])) : bf16_hi(v[u][c]);
        v[u][c] = pack_bf16x2(bf16_lo(rv[u][c]) + t0, bf16_hi(rv[u][c]) + t1);
      }
      *reinterpret_cast<u32x4*>(out_lane + (it0 + u) * out_step) = v[u];
    }
  };
  const bool interior = m_base + 64 <= p.M && n_base + 128 <= p.N;  // wave-uniform
  if (RESID && interior) {
    u32x4 rv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) rv[u] = *reinterpret_cast<const u32x4*>(res_lane + u * res_step);
    stage_half(0);
    rows8_prefetched(0, rv);
#pragma unroll
    for (int u = 0; u < 8; ++u) rv[u] = *reinterpret_cast<const u32x4*>(res_lane + (8 + u) * res_step);
    stage_half(1);
    rows8_prefetched(8, rv);
    return;
  }
#pragma unroll
  for (int tm = 0; tm < 2; ++tm) {
    stage_half(tm);
    if (interior)
      rows8(tm * 8, false);
    else
      rows8(tm * 8, true);
  }
}

// s_waitcnt immediate for vmcnt(vm) and lgkmcnt(lgkm) (15 = do not wait), expcnt left alone
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (lgkm << 8); }

// WM = waves along m, MT = 16-token MFMA columns per wave; the wave tile is 128 (n) x 16 MT (m):
//   WM 4, MT 4: 256 x 256 tile, eight waves of 128 x 64, two per SIMD;
//   WM 2, MT 4: 256 (n) x 128 (m) tile, four waves, for problems with so few 256 x 256 tiles that half the compute
//               units would idle.
// (WM 2, MT 8 -- four waves of 128 x 128 on a 256 x 256 tile, accumulators in 256 AccVGPRs -- compiles and passes
// the same tests; it is not instantiated, see above.)
// Same K order in every form, so a row's bits do not depend on which of them computed it.
// EXT: a second segment of the reduction axis may follow the first (GemmArgs::K2); a variant of its own, because the
// cross-over's bookkeeping costs the plain loop 3 %.
template <bool RESID, bool QK, int WM = 4, int MT = 4, bool EXT = false>
__global__ __launch_bounds__(128 * WM) void fp8_gemm_kernel(GemmPair q) {
  constexpr int PW = 16 / WM;  // 1 KiB pieces of a W unit (256 rows) per wave
  constexpr int PA = MT;       // 1 KiB pieces of an A unit (32 WM MT rows) per wave
  constexpr int TM = WM * MT * 16;  // token rows of the tile
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // Both problems' arguments are fetched together with the tile counts, in one round of scalar loads, and the
  // selected set is pinned in front of the early exit: left alone, the compiler sinks the argument loads below
  // the exit branch, behind the wait for the counts, and every workgroup starts with two dependent round trips.
  int L = logical_tile(blockIdx.x, q.total);
  const bool second = L >= q.total0;
  const GemmArgs p = pick(q, second);
  asm volatile("" ::"s"(p.a), "s"(p.w), "s"(p.lda), "s"(p.ldw), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.tiles_m),
               "s"(p.tiles_n));
  if (L >= q.total) return;
  if (second) L -= q.total0;
  int tm, tn;
  tile_of(L, p.tiles_m, p.tiles_n, tm, tn);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;            // 0..2 WM - 1
  const int wn = wave / WM, wm = wave % WM;
  const int m0 = tm * TM, n0 = tn * BN;

  // async loads: per unit a wave issues one instruction per 8 rows of its share
  const int ld_r = lane >> 3, ld_p = lane & 7;
  uint32_t w_off[PW], a_off[PA];
#pragma unroll
  for (int i = 0; i < PW; ++i) {
    const int row = (wave * PW + i) * 8 + ld_r;
    const int c = ld_p ^ ((row >> 1) & 7);
    w_off[i] = (uint32_t)(min(n0 + row, p.N - 1) - n0) * (uint32_t)p.ldw + c * 16;
  }
#pragma unroll
  for (int i = 0; i < PA; ++i) {
    const int row = (wave * PA + i) * 8 + ld_r;
    const int c = ld_p ^ ((row >> 1) & 7);
    a_off[i] = (uint32_t)(min(m0 + row, p.M - 1) - m0) * (uint32_t)p.lda + c * 16;
  }
  const uint8_t* w_base = p.w + (int64_t)n0 * p.ldw;
  const uint8_t* a_base = p.a + (int64_t)m0 * p.lda;
  // Units [0, nu1) come from (a, w), units [nu1, nu) from the optional second segment (a2, w2), whose rows are the
  // same rows at other leading dimensions: the per-lane offsets are re-formed once, when the loads cross over.
  const int nu1 = p.K / UK;
  const int nu = EXT ? nu1 + p.K2 / UK : nu1;
  const uint8_t* w2_base = p.w2 + (int64_t)n0 * p.ldw2 - (int64_t)nu1 * UK;  // so that unit j sits at base + j * UK
  const uint8_t* a2_base = p.a2 + (int64_t)m0 * p.lda2 - (int64_t)nu1 * UK;
  auto cross_over = [&](int op) {
    if (op == 0) {
#pragma unroll
      for (int i = 0; i < PW; ++i) {
        const int row = (wave * PW + i) * 8 + ld_r;
        const int c = ld_p ^ ((row >> 1) & 7);
        w_off[i] = (uint32_t)(min(n0 + row, p.N - 1) - n0) * (uint32_t)p.ldw2 + c * 16;
      }
    } else {
#pragma unroll
      for (int i = 0; i < PA; ++i) {
        const int row = (wave * PA + i) * 8 + ld_r;
        const int c = ld_p ^ ((row >> 1) & 7);
        a_off[i] = (uint32_t)(min(m0 + row, p.M - 1) - m0) * (uint32_t)p.lda2 + c * 16;
      }
    }
  };
  // The async loads are issued as assembly in the scalar-base + 32-bit-lane-offset form: the builtin takes a
  // 64-bit per-lane address, and eight of those (plus their increments) are sixteen registers the eight-wave
  // form, at 256 per wave, does not have.  M0 carries the LDS destination; nothing else here uses M0.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)smem;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  auto issue_load = [&](int j, int op, int i) {
    const int slot = (2 * j + op) % NSLOT;
    j = min(j, nu - 1);
    if (EXT && i == 0 && j == nu1 && p.K2 > 0) cross_over(op);  // (pieces of a unit go out in order, units in order)
    const uint32_t dst = lds0 + slot * kUnitBytes + (wave_u * (op ? PA : PW) + i) * 1024;
    const uint8_t* ub = (EXT && j >= nu1 ? (op ? a2_base : w2_base) : (op ? a_base : w_base)) + (int64_t)j * UK;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(op ? a_off[i] : w_off[i]), "s"(ub), "s"(dst)
                 : "memory", "m0");
  };
#pragma clang diagnostic pop

  // Operand fragments of v_mfma_f32_16x16x128_f8f6f4: lane (q = lane / 16, i = lane % 16) holds the 32 K-bytes
  // [32q, 32q + 32) of row i of a 16-row tile, i.e. chunks 2q and 2q + 1 of a 128-byte unit row: one MFMA consumes
  // a whole unit row of either operand.  A wave's tile is 8 W tiles x MT A tiles = 8 MT MFMAs per unit.  W tile i
  // feeds MFMAs i MT .. i MT + MT - 1 only, so W fragments live in a ring of four register octets and are read
  // three tiles ahead of their use; the A fragments, which every W tile meets, are double-buffered per unit.
  const int q16 = lane >> 4, i16 = lane & 15;
  const int w_row = wn * 128 + i16;
  const int a_row = wm * (MT * 16) + i16;
  i32x4 wr[4][2];      // [ring slot][half]
  i32x4 ar[2][MT][2];  // [buffer][tile][half]
  // Read addresses: a lane constant per half and operand (a tile adds 16 rows = 2048 bytes as an immediate: the
  // swizzle of row + 16t equals that of row) plus the ring slot of the unit.  The sums live in registers that are
  // re-pointed once per unit -- wa[k]: W of units of parity k (the unit being computed and the next one alternate
  // between the two), aa: A of the next unit -- instead of being formed at each of a unit's 16 + 2 MT reads.
  uint32_t w_la[2], a_la[2], wa[2][2], aa[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    w_la[half] = (uint32_t)unit_off(w_row, q16 * 2 + half);
    a_la[half] = (uint32_t)unit_off(a_row, q16 * 2 + half);
  }
  auto point_w = [&](int k, int j) {  // wa[k] -> W of unit j
    uint32_t slot_off = (uint32_t)(((2 * j) % NSLOT) * kUnitBytes);
    asm volatile("" : "+s"(slot_off));
    wa[k][0] = w_la[0] + slot_off;
    wa[k][1] = w_la[1] + slot_off;
  };
  auto point_a = [&](int j) {  // aa -> A of unit j
    uint32_t slot_off = (uint32_t)(((2 * j + 1) % NSLOT) * kUnitBytes);
    asm volatile("" : "+s"(slot_off));
    aa[0] = a_la[0] + slot_off;
    aa[1] = a_la[1] + slot_off;
  };
  auto read_w = [&](int k, int tile, int half) {   // W tile `tile` (0..7) of the unit wa[k] points at
    wr[tile & 3][half] = *reinterpret_cast<const i32x4*>(smem + wa[k][half] + tile * 2048);
  };
  auto read_a = [&](int buf, int tile, int half) {
    ar[buf][tile][half] = *reinterpret_cast<const i32x4*>(smem + aa[half] + tile * 2048);
  };

  f32x4 acc[8][MT];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  auto mfma_one = [&](int buf, int i, int t) {   // W tile i x A tile t
    const i32x4 w0 = wr[i & 3][0], w1 = wr[i & 3][1], a0 = ar[buf][t][0], a1 = ar[buf][t][1];
    const i32x8 vw = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
    const i32x8 va = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    acc[i][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vw, va, acc[i][t], 0, 0, 0, 0, 0, 0);
  };

  // Operands of the epilogue.  Columns >= N and rows >= M are never stored, so their addresses are clamped
  // instead of predicated (a lane-predicated load is not batched with its neighbours).
  EpiOperands<MT> epi;
  float w_scale_raw = 1.0f;
  auto load_epi = [&]() {  // loads only: whatever uses a loaded value would wait for it on the spot
    const int n_base = n0 + wn * 128, m_base = m0 + wm * (MT * 16);
    if (p.w_scale) w_scale_raw = *p.w_scale;
    if (p.bias) {
#pragma unroll
      for (int t = 0; t < 8; ++t)
        epi.bias[t] = *reinterpret_cast<const u32x2*>(p.bias + min(n_base + t * 16 + 4 * q16, p.N - 4));
    } else {
#pragma unroll
      for (int t = 0; t < 8; ++t) epi.bias[t] = u32x2{0, 0};
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
      epi.sc[t] = p.a_scale ? p.a_scale[min(m_base + t * 16 + i16, p.M - 1)] : 1.0f;
  };

  // One unit = 128 bytes of K = 8 MT MFMAs per wave (slot s: W tile s / MT, A tile s % MT); the A fragments of
  // unit j sit in ar[buf], its first three W tiles in the ring, wa[par] points at its W slot and wa[par ^ 1] at the
  // next unit's.  Between the MFMAs the wave reads W tile s / MT + 3 (in the first two slots of a tile, one half
  // each), which from slot 5 MT on is a tile of unit j + 1, reads the A fragments of unit j + 1 into the other
  // buffer (2 MT slots from 5 MT + 2 on), issues its async loads of W unit j + 2 (slots below 4 MT) and of A unit
  // j + 2 (after slot 5 MT).  Slot 5 MT opens with the unit's one synchronisation point: every load but the W pieces
  // just issued has landed (unit j + 1 is complete), every wave has finished reading unit j (its last W tile was
  // read in slots 4 MT and 4 MT + 1), so unit j's two ring slots can be overwritten -- A unit j + 2 takes the one
  // W unit j had, W unit j + 3 (a unit later) the one A unit j had.
  // `loads` = false for the last two units (nothing is left to fetch); `last` = true for the very last: no next
  // unit to read from, and the registers its fragments would occupy take the epilogue's operands instead.
  constexpr int NS = 8 * MT, kSync = 5 * MT;
  auto unit = [&](int j, int par, bool loads, bool last) {
    const int buf = par;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int i = s / MT, t = s % MT;
      if (s == kSync) {
        if (loads)
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(PW, 0));  // all but the W pieces of this unit; lgkmcnt(0)
        else
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));   // vmcnt(0) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        if (!last) {
          point_w(par, j + 2);  // this unit's W slot has been read for the last time: on to the unit after next
          point_a(j + 1);
        }
      }
      mfma_one(buf, i, t);
      if (t < 2) {
        const int tile = i + 3;
        if (tile < 8)
          read_w(par, tile, t);
        else if (!last)
          read_w(par ^ 1, tile - 8, t);
      }
      if (last) {
        if (s == 6 * MT) load_epi();  // the W ring is down to its last two tiles: their neighbours take the operands
      } else {
        if (s >= kSync + 2 && s < kSync + 2 + 2 * MT) read_a(buf ^ 1, (s - kSync - 2) >> 1, (s - kSync - 2) & 1);
        if (loads) {
          constexpr int kWStride = 4 * MT / PW;
          if (s < 4 * MT && (s % kWStride) == kWStride - 1) issue_load(j + 2, 0, s / kWStride);
          if (s > kSync && (s - kSync - 1) % 3 == 0 && (s - kSync - 1) / 3 < PA) issue_load(j + 2, 1, (s - kSync - 1) / 3);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int i = 0; i < ((u & 1) ? PA : PW); ++i) issue_load(u >> 1, u & 1, i);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(PW + PA, 15));  // all but W and A unit 1: W and A unit 0 have landed
  __builtin_amdgcn_s_barrier();
  // Parity of unit j: (j + nu) % 2, so that the last unit always has parity 1 and the one before it parity 0
  // whatever the unit count; it selects the A buffer and which of wa[] points at the unit.
  point_a(0);
  if (nu & 1) {
    point_w(1, 0);
    point_w(0, 1);
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      read_w(1, t, 0);
      read_w(1, t, 1);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      read_a(1, t, 0);
      read_a(1, t, 1);
    }
  } else {
    point_w(0, 0);
    point_w(1, 1);
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      read_w(0, t, 0);
      read_w(0, t, 1);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      read_a(0, t, 0);
      read_a(0, t, 1);
    }
  }

  {
    int j = 0;
    const int n_loading = nu >= 2 ? nu - 2 : 0;  // units that still have loads to issue
    if (n_loading & 1) {
      unit(0, 1, true, false);
      j = 1;
    }
    for (; j < n_loading; j += 2) {
      unit(j, 0, true, false);
      unit(j + 1, 1, true, false);
    }
    if (nu >= 2) unit(nu - 2, 0, false, false);
    unit(nu - 1, 1, false, true);
  }
  // No barrier in front of the epilogue: the last unit's synchronisation point came after every wave's final
  // fragment reads and after every async load had landed, so the ring is dead from there on and a wave may
  // overwrite its private staging region as soon as its own MFMAs are issued.
  // (compiler-only fence: without it the epilogue's residual loads are hoisted into the last unit, where every
  // register is taken, and the accumulators they displace are spilled)
  asm volatile("" ::: "memory");
#pragma unroll
  for (int t = 0; t < MT; ++t) epi.sc[t] *= w_scale_raw;
  uint8_t* const stage = smem + wave * kEpiBytesPerWave;
  store_ct_lds<RESID, QK, MT, 0>(p, acc, epi, stage, n0 + wn * 128, m0 + wm * (MT * 16), lane);
  if constexpr (MT == 8)
    store_ct_lds<RESID, QK, MT, 1>(p, acc, epi, stage, n0 + wn * 128, m0 + wm * (MT * 16) + 64, lane);
}

// ------------------------------------------------------------------------------------------
// Generic kernel: any K % 16 == 0 (zero-filled K tail), any N / alignment (scalar stores where the
// 8-byte path does not apply).  Register-staged loads, one LDS stage; used for the few odd shapes.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fp8_gemm_ragged_k_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int tm, tn;
  bool valid;
  tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn, valid);
  if (!valid) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wn = wave >> 1, wm = wave & 1;
  const int g = lane >> 5, li = lane & 31;
  const int m0 = tm * BM, n0 = tn * BN;
  const int kchunks = p.K >> 4;
  const int st_c = tid & 7, st_r = tid >> 3;
  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  uint8_t* sW = smem;
  uint8_t* sA = smem + kTileBytes;
  const int nk = (p.K + BK - 1) / BK;
  for (int kt = 0; kt < nk; ++kt) {
    const bool in = (kt * 8 + st_c) < kchunks;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = st_r + 32 * i;
      u32x4 wv = {0, 0, 0, 0}, av = {0, 0, 0, 0};
      if (in) {
        wv = *reinterpret_cast<const u32x4*>(p.w + (int64_t)min(n0 + row, p.N - 1) * p.ldw +
                                             (int64_t)kt * BK + st_c * 16);
        av = *reinterpret_cast<const u32x4*>(p.a + (int64_t)min(m0 + row, p.M - 1) * p.lda +
                                             (int64_t)kt * BK + st_c * 16);
      }
      *reinterpret_cast<u32x4*>(sW + lds_off(row, st_c)) = wv;
      *reinterpret_cast<u32x4*>(sA + lds_off(row, st_c)) = av;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      i32x8 fw[4], fa[4];
      const int c0 = ks * 4 + g * 2;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int rw = wn * 128 + t * 32 + li, ra = wm * 128 + t * 32 + li;
        const i32x4 w_lo = *reinterpret_cast<const i32x4*>(sW + lds_off(rw, c0));
        const i32x4 w_hi = *reinterpret_cast<const i32x4*>(sW + lds_off(rw, c0 + 1));
        const i32x4 a_lo = *reinterpret_cast<const i32x4*>(sA + lds_off(ra, c0));
        const i32x4 a_hi = *reinterpret_cast<const i32x4*>(sA + lds_off(ra, c0 + 1));
        fw[t] = i32x8{w_lo.x, w_lo.y, w_lo.z, w_lo.w, w_hi.x, w_hi.y, w_hi.z, w_hi.w};
        fa[t] = i32x8{a_lo.x, a_lo.y, a_lo.z, a_lo.w, a_hi.x, a_hi.y, a_hi.z, a_hi.w};
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fw[i], fa[j], acc[i][j], 0, 0,
                                                                      0, 0, 0, 0);
    }
    __syncthreads();
  }
  store_ct(p, acc, n0 + wn * 128, m0 + wm * 128, g, li);
}

// Small-M path (M <= 8): HBM-bound on the weight read (the M=1 conditioning projections).
// One wavefront owns four output rows; per K chunk of 1 KiB a lane fetches 16 weight bytes of
// each row (four independent loads in flight) and reuses its 16 activation bytes per token.
// fp32 FMA over the dequantised bytes; the per-row scale form serves several Linear layers
// stacked into one weight matrix.
__device__ __forceinline__ void dequant16(const u32x4& v, float* f) {
  // v_cvt_pk_f32_fp8: two OCP e4m3 bytes of a dword -> two fp32, one VALU instruction per pair
  // (a bit-twiddling decode costs ~12 per byte and made this kernel VALU-bound)
  typedef float f32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[w], false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[w], true);
    f[4 * w + 0] = lo[0];
    f[4 * w + 1] = lo[1];
    f[4 * w + 2] = hi[0];
    f[4 * w + 3] = hi[1];
  }
}

template <int MT>
__global__ __launch_bounds__(256) void fp8_gemv_kernel(GemmArgs p) {
  const int lane = threadIdx.x & 63;
  const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4;
  if (n0 >= p.N) return;
  const int kchunks = p.K >> 4;
  float acc[4][MT];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;
  const u32x4* wr[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) wr[r] = reinterpret_cast<const u32x4*>(p.w + (int64_t)min(n0 + r, p.N - 1) * p.ldw);
  for (int c = lane; c < kchunks; c += 64) {
    u32x4 wv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) wv[r] = __builtin_nontemporal_load(wr[r] + c);
    float af[MT][16];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const u32x4 av = *reinterpret_cast<const u32x4*>(p.a + (int64_t)min(m, p.M - 1) * p.lda + c * 16);
      dequant16(av, af[m]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float wf[16];
      dequant16(wv[r], wf);
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int b = 0; b < 16; ++b) acc[r][m] += wf[b] * af[m][b];
    }
  }
  const float ws = p.w_scale ? *p.w_scale : 1.0f;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = n0 + r;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float s = wave_sum(acc[r][m]);
      if (lane == 0 && n < p.N && m < p.M) {
        const float as = p.a_scale ? p.a_scale[m] : 1.0f;
        const float wsn = p.w_row_scale ? p.w_row_scale[n] : ws;
        const float bj = p.bias ? bf16_bits_to_f32(p.bias[n]) : 0.f;
        float r = s * (as * wsn) + bj;
        if (p.resid) r = residual_combine(p, round_bf16(r), m, n);
        p.out[(int64_t)m * p.ldo + n] = (uint16_t)f32_to_bf16_bits(r);
      }
    }
  }
}

static int launch_gemv(const GemmArgs& p, hipStream_t st) {
  const dim3 grid((unsigned)((p.N + 15) / 16)), block(256);
  if (p.M == 1) fp8_gemv_kernel<1><<<grid, block, 0, st>>>(p);
  else if (p.M == 2) fp8_gemv_kernel<2><<<grid, block, 0, st>>>(p);
  else if (p.M <= 4) fp8_gemv_kernel<4><<<grid, block, 0, st>>>(p);
  else fp8_gemv_kernel<8><<<grid, block, 0, st>>>(p);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

}  // namespace dsx

static int gemm_set_attributes() {
  using namespace dsx;
  static PerDeviceOnce once;
  return per_device_once(once, [](int) {
    const void* kernels[] = {
        (const void*)fp8_gemm_kernel<false, false, 4, 4>,       (const void*)fp8_gemm_kernel<true, false, 4, 4>,
        (const void*)fp8_gemm_kernel<false, true, 4, 4>,        (const void*)fp8_gemm_kernel<false, false, 2, 4>,
        (const void*)fp8_gemm_kernel<true, false, 2, 4>,        (const void*)fp8_gemm_kernel<false, true, 2, 4>,
        (const void*)fp8_gemm_kernel<false, false, 4, 4, true>, (const void*)fp8_gemm_kernel<true, false, 4, 4, true>,
        (const void*)fp8_gemm_kernel<false, true, 4, 4, true>,  (const void*)fp8_gemm_kernel<false, false, 2, 4, true>,
        (const void*)fp8_gemm_kernel<true, false, 2, 4, true>,  (const void*)fp8_gemm_kernel<false, true, 2, 4, true>};
    for (const void* k : kernels)
      if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kMainLdsBytes) != hipSuccess)
        return (int)DSX_ELAUNCH;
    if (hipFuncSetAttribute((const void*)fp8_gemm_ragged_k_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            kStageBytes) != hipSuccess)
      return (int)DSX_ELAUNCH;
    return (int)DSX_OK;
  });
}

// Fills the tile counts and says whether the problem can run on the main 256x256 kernel.
static bool gemm_main_kernel_ok(dsx::GemmArgs& p) {
  using namespace dsx;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const bool vec_ok = ((p.ldo & 7) == 0) && ((p.N & 7) == 0) && (((uintptr_t)p.out & 15) == 0) &&
                      (!p.bias || ((uintptr_t)p.bias & 7) == 0) &&
                      (!p.resid || ((((uintptr_t)p.resid & 15) == 0) && ((p.ldr & 7) == 0) &&
                                    (((uintptr_t)p.gate & 15) == 0) && ((p.gate_sb & 7) == 0)));
  return p.M > 8 && !p.w_row_scale && (p.K % 128) == 0 && vec_ok;
}

constexpr int kHalfTileThreshold = 128;

// The instantiation for one launch: epilogue kind of the first problem (pairs agree on it), waves along m, and
// whether either problem continues its reduction axis in a second segment.
template <int WM>
static void launch_form(const dsx::GemmPair& q, const dsx::GemmArgs& p0, bool ext, int grid, hipStream_t st) {
  using namespace dsx;
  const dim3 g((unsigned)grid), b(128 * WM);
#define DSX_GO(R, Q)                                                                   \
  do {                                                                                 \
    if (ext)                                                                           \
      fp8_gemm_kernel<R, Q, WM, 4, true><<<g, b, kMainLdsBytes, st>>>(q);              \
    else                                                                               \
      fp8_gemm_kernel<R, Q, WM, 4, false><<<g, b, kMainLdsBytes, st>>>(q);             \
  } while (0)
  if (p0.resid)
    DSX_GO(true, false);
  else if (p0.qk_heads > 0)
    DSX_GO(false, true);
  else
    DSX_GO(false, false);
#undef DSX_GO
}

// One launch of the main kernel over one or two problems (of the same kind: plain, residual or qk epilogue).
static int launch_main(const dsx::GemmArgs& p0, const dsx::GemmArgs* p1, hipStream_t st) {
  using namespace dsx;
  GemmPair q;
  q.p[0] = p0;
  q.p[1] = p1 ? *p1 : p0;
  q.total0 = p0.tiles_m * p0.tiles_n;
  q.total = q.total0 + (p1 ? p1->tiles_m * p1->tiles_n : 0);
  const bool ext = p0.K2 > 0 || (p1 && p1->K2 > 0);
  // At most half the compute units' worth of 256 x 256 tiles (MI355X: 256): tiles of 128 token rows fill twice
  // as many, and the four-wave form of the kernel runs them (same wave tile and K order: same bits).
  if (q.total <= kHalfTileThreshold) {
    q.p[0].tiles_m = (p0.M + 127) / 128;
    q.p[1].tiles_m = p1 ? (p1->M + 127) / 128 : q.p[0].tiles_m;
    q.total0 = q.p[0].tiles_m * p0.tiles_n;
    q.total = q.total0 + (p1 ? q.p[1].tiles_m * p1->tiles_n : 0);
    const int grid = ((q.total + 7) / 8) * 8;
    launch_form<2>(q, p0, ext, grid, st);
    return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
  }
  const int grid = ((q.total + 7) / 8) * 8;
  launch_form<4>(q, p0, ext, grid, st);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

static int gemm_dispatch(dsx::GemmArgs& p, int64_t M, int64_t N, int64_t K, hipStream_t st) {
  using namespace dsx;
  (void)N; (void)K;
  if (M <= 8) {
    p.tiles_m = p.tiles_n = 0;
    return launch_gemv(p, st);
  }
  if (p.w_row_scale) return DSX_EBADSHAPE;
  if (gemm_set_attributes() != DSX_OK) return DSX_ELAUNCH;
  if (gemm_main_kernel_ok(p)) return launch_main(p, nullptr, st);
  const int total = p.tiles_m * p.tiles_n;
  const int grid = ((total + 7) / 8) * 8;
  fp8_gemm_ragged_k_kernel<<<dim3((unsigned)grid), dim3(256), kStageBytes, st>>>(p);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

static int gemm_fill(dsx::GemmArgs& p, const void* a, int64_t lda, const void* w, int64_t ldw,
                     const float* a_scale, const float* w_scale, const void* bias, void* out, int64_t ldo,
                     int64_t M, int64_t N, int64_t K) {
  if (M == 0 && w) {  // an empty batch: nothing to compute, no activation or output buffer needed
    p.M = 0;
    return (N <= 0 || K <= 0) ? DSX_EBADSHAPE : DSX_OK;
  }
  if (!a || !w || !out) return DSX_ENULL;
  if (M < 0 || N <= 0 || K <= 0 || (K & 15) || lda < K || ldw < K || ldo < N) return DSX_EBADSHAPE;
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return DSX_EBADSHAPE;
  // The kernels form per-lane operand offsets row * ld (row < 256) in 32 bits and count tiles in an int.
  if (lda >= (1 << 24) || ldw >= (1 << 24)) return DSX_EBADSHAPE;
  if (((M + 63) / 64) * ((N + 63) / 64) > (1ll << 30)) return DSX_EBADSHAPE;
  if ((lda & 15) || (ldw & 15) || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || ((uintptr_t)out & 1) ||
      ((uintptr_t)bias & 1))
    return DSX_EALIGN;
  p.a = (const uint8_t*)a;
  p.w = (const uint8_t*)w;
  p.a_scale = a_scale;
  p.w_scale = w_scale;
  p.bias = (const uint16_t*)bias;
  p.out = (uint16_t*)out;
  p.lda = lda;
  p.ldw = ldw;
  p.ldo = ldo;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.resid = nullptr;
  p.gate = nullptr;
  p.ldr = p.gate_sb = 0;
  p.rows_per_batch = 1;
  p.w_row_scale = nullptr;
  p.qk_wq = p.qk_wk = nullptr;
  p.rope = nullptr;
  p.rope_sb = 0;
  p.rope_pos0 = p.qk_heads = 0;
  p.qk_eps = 0.f;
  p.a2 = p.w2 = nullptr;
  p.lda2 = p.ldw2 = 0;
  p.K2 = 0;
  return DSX_OK;
}

extern "C" int dsx_fp8_gemm(const void* a, int64_t lda, const void* w, int64_t ldw,
                            const float* a_scale, const float* w_scale, const void* bias, void* out,
                            int64_t ldo, int64_t M, int64_t N, int64_t K, void* stream) {
  dsx::GemmArgs p;
  const int rc = gemm_fill(p, a, lda, w, ldw, a_scale, w_scale, bias, out, ldo, M, N, K);
  if (rc != DSX_OK || M == 0) return rc;
  return gemm_dispatch(p, M, N, K, (hipStream_t)stream);
}

extern "C" int dsx_fp8_gemm_gated_residual(const void* a, int64_t lda, const void* w, int64_t ldw,
                                           const float* a_scale, const float* w_scale, const void* bias,
                                           const void* resid, int64_t ldr, const void* gate, int64_t gate_sb,
                                           int64_t rows_per_batch, void* out, int64_t ldo, int64_t M,
                                           int64_t N, int64_t K, void* stream) {
  dsx::GemmArgs p;
  const int rc = gemm_fill(p, a, lda, w, ldw, a_scale, w_scale, bias, out, ldo, M, N, K);
  if (rc != DSX_OK || M == 0) return rc;
  if (!resid) return DSX_ENULL;
  if (ldr < N || rows_per_batch <= 0 || rows_per_batch > (1 << 30)) return DSX_EBADSHAPE;
  if (((uintptr_t)resid & 1) || ((uintptr_t)gate & 1)) return DSX_EALIGN;
  p.resid = (const uint16_t*)resid;
  p.gate = (const uint16_t*)gate;
  p.ldr = ldr;
  p.gate_sb = gate_sb;
  p.rows_per_batch = (int)rows_per_batch;
  return gemm_dispatch(p, M, N, K, (hipStream_t)stream);
}

extern "C" int dsx_fp8_gemv_rowscale(const void* a, int64_t lda, const void* w, int64_t ldw,
                                     const float* a_scale, const float* w_row_scale, const void* bias,
                                     void* out, int64_t ldo, int64_t M, int64_t N, int64_t K,
                                     void* stream) {
  dsx::GemmArgs p;
  const int rc = gemm_fill(p, a, lda, w, ldw, a_scale, nullptr, bias, out, ldo, M, N, K);
  if (rc != DSX_OK || M == 0) return rc;
  if (M > 8) return DSX_EBADSHAPE;
  if (!w_row_scale) return DSX_ENULL;
  p.w_row_scale = w_row_scale;
  return gemm_dispatch(p, M, N, K, (hipStream_t)stream);
}

static int problem_fill(dsx::GemmArgs& p, const dsx_gemm_problem& d) {
  int rc = gemm_fill(p, d.a, d.lda, d.w, d.ldw, d.a_scale, d.w_scale, d.bias, d.out, d.ldo, d.M, d.N, d.K);
  if (rc != DSX_OK) return rc;
  if (d.resid) {
    if (d.ldr < d.N || d.rows_per_batch <= 0 || d.rows_per_batch > (1 << 30)) return DSX_EBADSHAPE;
    if (((uintptr_t)d.resid & 1) || ((uintptr_t)d.gate & 1)) return DSX_EALIGN;
    p.resid = (const uint16_t*)d.resid;
    p.gate = (const uint16_t*)d.gate;
    p.ldr = d.ldr;
    p.gate_sb = d.gate_sb;
    p.rows_per_batch = (int)d.rows_per_batch;
  } else if (d.gate) {
    return DSX_ENULL;  // a gate without a residual is not an operation of the path
  }
  if (d.qk_heads != 0) {
    // the q/k epilogue lives in the 256x256-tile kernel only, whose waves own whole 128-column heads
    if (d.qk_heads < 0 || d.resid || d.M <= 0 || 2 * (int64_t)d.qk_heads * 128 > d.N) return DSX_EBADSHAPE;
    if (d.rows_per_batch <= 0 || d.rows_per_batch > (1 << 30)) return DSX_EBADSHAPE;
    if (((uintptr_t)d.q_norm_w & 15) || ((uintptr_t)d.k_norm_w & 15) || ((uintptr_t)d.rope & 15) || (d.rope_sb & 3))
      return DSX_EALIGN;
    if (d.rope) {
      const int64_t batches = (d.M + d.rows_per_batch - 1) / d.rows_per_batch;
      const int64_t last = d.rope_pos0 + (d.M < d.rows_per_batch ? d.M : d.rows_per_batch);
      if (d.rope_pos0 < 0 || d.rope_pos0 > (1 << 30) || d.rope_rows < last) return DSX_EBADSHAPE;
      if (batches > 1 && d.rope_sb != 0 && d.rope_sb < d.rope_rows * 128) return DSX_EBADSHAPE;
    }
    p.qk_wq = (const uint16_t*)d.q_norm_w;
    p.qk_wk = (const uint16_t*)d.k_norm_w;
    p.rope = d.rope;
    p.rope_sb = d.rope_sb;
    p.rope_pos0 = (int)d.rope_pos0;
    p.qk_heads = d.qk_heads;
    p.qk_eps = d.norm_eps;
    p.rows_per_batch = (int)d.rows_per_batch;
    if (!gemm_main_kernel_ok(p)) return DSX_EBADSHAPE;
  }
  if (d.K_ext != 0) {
    // the second segment of the reduction axis exists in the tile kernel only; its unit count and the kernel's
    // prologue (two units of the first segment) bound the shapes
    if (d.K_ext < 0 || d.K_ext > (1 << 30) || (d.K_ext % 128) || d.K < 256 || d.M <= 0) return DSX_EBADSHAPE;
    if (!d.a_ext || !d.w_ext) return DSX_ENULL;
    if (d.lda_ext < d.K_ext || d.ldw_ext < d.K_ext || d.lda_ext >= (1 << 24) || d.ldw_ext >= (1 << 24)) return DSX_EBADSHAPE;
    if ((d.lda_ext & 15) || (d.ldw_ext & 15) || ((uintptr_t)d.a_ext & 15) || ((uintptr_t)d.w_ext & 15)) return DSX_EALIGN;
    p.a2 = (const uint8_t*)d.a_ext;
    p.w2 = (const uint8_t*)d.w_ext;
    p.lda2 = d.lda_ext;
    p.ldw2 = d.ldw_ext;
    p.K2 = (int)d.K_ext;
    if (!gemm_main_kernel_ok(p)) return DSX_EBADSHAPE;
  }
  return DSX_OK;
}

extern "C" int dsx_fp8_gemm_grouped(const dsx_gemm_problem* problems, int count, void* stream) {
  if (count < 0 || count > DSX_GEMM_GROUP_MAX) return DSX_EBADSHAPE;
  if (count == 0) return DSX_OK;
  if (!problems) return DSX_ENULL;
  dsx::GemmArgs args[DSX_GEMM_GROUP_MAX];
  for (int i = 0; i < count; ++i) {  // validate everything before anything is launched
    const int rc = problem_fill(args[i], problems[i]);
    if (rc != DSX_OK) return rc;
  }
  hipStream_t st = (hipStream_t)stream;
  if (gemm_set_attributes() != DSX_OK) return DSX_ELAUNCH;
  bool main_ok[DSX_GEMM_GROUP_MAX];
  for (int i = 0; i < count; ++i) main_ok[i] = args[i].M > 0 && gemm_main_kernel_ok(args[i]);
  int i = 0;
  while (i < count) {
    if (args[i].M == 0) { ++i; continue; }
    // pair neighbours that both run on the main kernel and agree on having a residual
    if (i + 1 < count && main_ok[i] && main_ok[i + 1] && (args[i].resid != nullptr) == (args[i + 1].resid != nullptr) &&
        (args[i].qk_heads > 0) == (args[i + 1].qk_heads > 0)) {
      const int rc = launch_main(args[i], &args[i + 1], st);
      if (rc != DSX_OK) return rc;
      i += 2;
      continue;
    }
    const int rc = gemm_dispatch(args[i], args[i].M, args[i].N, args[i].K, st);
    if (rc != DSX_OK) return rc;
    ++i;
  }
  return DSX_OK;
}
