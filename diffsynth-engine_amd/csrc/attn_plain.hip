// Flash attention forward for gfx950 without fused pre-processing (q and k already normalised
// and rotated): head dim 128, bf16 operands, fp32 online softmax.
//
// MFMA formulation as in attn_fwd.hip (S^T = K Q^T, O^T += V^T P^T, one query per lane, so the
// softmax statistics are lane-local apart from one exchange between the two half-waves).
//
// Work split: one workgroup = 8 waves = 256 consecutive queries of one (batch, head); every wave
// owns 32 queries and needs ~230 VGPRs, so two waves share a SIMD and one workgroup fills a CU.
// While one wave of a SIMD works through exp2/convert/row-sum on the VALU, the other's MFMAs can
// keep the matrix pipe busy.  That costs one LDS operand read per MFMA, which the 256 B/clk LDS of
// CDNA4 carries at a quarter load.
//
//  * K and V blocks (64 keys) go HBM/L2 -> LDS with global_load_lds_dwordx4, four stages deep,
//    both stored row-major [key][128 d].  No staging registers, no transposing stores.
//  * The V^T operand (8 keys of one d per lane) is read from the row-major V tile with
//    ds_read_b64_tr_b16: in a 16-lane group, lane i receives element i%4 of the 8-byte datum
//    addressed by lanes i/4, i/4+4, i/4+8, i/4+12.  Source lane j therefore points at
//    V[key0 + j/4][d0 + 4*(j%4)], and the receiver gets 4 consecutive keys of d = d0 + i.
//  * Q is pre-multiplied by softmax_scale*log2(e) once, so P = exp2(S - m_ref) needs no multiply.
//    The reference m_ref stays 0 (no subtract either) unless a block maximum leaves [-64, 64] in
//    the first block or exceeds 64 later; after RMSNorm the log2-domain scores are bounded by
//    128*scale*log2(e) ~ 16.  Moving the reference rescales O and l, so the result is exact
//    softmax in every case.
//
// LDS swizzles: K rows (256 B): 16-byte chunk c of key r at c ^ (r & 15)  (ds_read_b128 by 32 rows);
//               V rows (256 B): chunk c of key r at c ^ ((r & 3) << 2)    (transposing 8-byte reads).
#include <algorithm>

#include "attn_internal.h"
#include "common.h"

namespace dsx {

namespace {

constexpr int QB = 256;  // queries per workgroup (8 waves x 32)
constexpr int KB = 64;   // keys per block
constexpr int HD = 128;
constexpr int kTile = KB * HD * 2;      // 16 KiB
constexpr int kStages = 4;
constexpr int kLdsBytes = 2 * kStages * kTile;  // K stages, then V stages
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kRescaleThreshold = 64.0f;  // log2 units

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
typedef short v4i16 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float pair_max(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

// Key-range split of the last, partly filled round of workgroups.  With U units on C compute units the
// last round keeps only U mod C of them busy; instead, the first `full_units` units run whole (one
// workgroup each) and the key axes of the remaining `tail_units` are laid end to end and cut into
// `pieces` equal runs of `len` 64-key blocks, one workgroup each, so that the last round ends everywhere
// at once.  A piece covers the end of one unit and/or the start of the next; each part leaves its
// unnormalised O, row sums and softmax references in a slot, and attn_merge_kernel combines the parts
// of a unit.
struct AttnSplit {
  int full_units, tail_units, pieces, len, max_parts;
  float* slots;
  int device_bound;  // the kernel reads p.qk_norm2_max and returns at once when the other variant is the one to run
};
constexpr int kSlotOFloats = QB * HD;               // O part: [dt][rq][wave][g][j][4]
constexpr int kSlotFloats = kSlotOFloats + 2 * QB;  // + row sums, + references

// normalised output of one lane: query `row`, d = dt*32 + 8*rq + 4g + 0..3 per (dt, rq)
__device__ __forceinline__ void store_output(const dsx_attn_params& p, int b, int h, int64_t row, int g,
                                             const f32x16 (&oacc)[4], float inv) {
  const int seg = row >= p.sq[0] ? 1 : 0;
  uint16_t* dst = (uint16_t*)p.o[seg] + (int64_t)b * p.o_sb[seg] + (int64_t)h * p.o_sh[seg] +
                  (row - (seg ? p.sq[0] : 0)) * p.o_ss[seg];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      u32x2 w;
      w.x = pack_bf16x2(oacc[dt][4 * rq + 0] * inv, oacc[dt][4 * rq + 1] * inv);
      w.y = pack_bf16x2(oacc[dt][4 * rq + 2] * inv, oacc[dt][4 * rq + 3] * inv);
      *reinterpret_cast<u32x2*>(dst + dt * 32 + 8 * rq + 4 * g) = w;
    }
}

// SCAN = false: the caller has bounded every |score| (log2 domain) by kRescaleThreshold, so the softmax
// reference can stay 0 for the whole row and the per-block maximum is not computed at all.
// SPLIT = false: every workgroup runs one whole unit (sp.full_units = all of them); the loop over parts
// and the variable key range fold away.
// QPRE = true: q still needs its RMSNorm (p.q_norm_w) and / or RoPE (p.rope); they are applied to the
// workgroup's 256 query rows as they are loaded, which is free (each q row is read exactly once).  K is
// read by every query block of its head, so the same work on k belongs in a one-off pass before this kernel.
template <bool SCAN, bool SPLIT, bool QPRE>
__global__ __launch_bounds__(512) void attn_plain_kernel(dsx_attn_params p, AttnSplit sp) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  if (sp.device_bound) {
    // Both variants were launched; the two device floats say which one works.  Not bounded (Inf and NaN
    // included, for which the comparison is false) means the variant with the running maximum.
    const float a = p.qk_norm2_max[0], b = p.qk_norm2_max[1];
    const bool bounded = sqrtf(a) * sqrtf(b) * p.softmax_scale * (kLog2e * 1.02f) <= kRescaleThreshold;
    if (bounded == SCAN) return;
  }
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;  // 0..7
  const int g = lane >> 5, li = lane & 31;
  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of (batch, head,
  // query block) units so that the query blocks of one head share that head's K/V through ONE L2
  // (with a plain 3-D grid every XCD ends up fetching every head's K and V).
  const int nqb = (int)((p.sq[0] + p.sq[1] + QB - 1) / QB);
  const int64_t Sq = p.sq[0] + p.sq[1];
  const int64_t Skv = p.skv[0] + p.skv[1];
  const int nkb = (int)((Skv + KB - 1) / KB);
  // what this workgroup does: one whole unit, or one piece of the split tail = up to two parts of units
  int nparts = 1, part_unit[2], part_kb0[2], part_kb1[2];
  const int full8 = (sp.full_units + 7) & ~7;
  if (!SPLIT || (int)blockIdx.x < full8) {
    part_unit[0] = (int)(blockIdx.x & 7) * (full8 >> 3) + (int)(blockIdx.x >> 3);
    if (part_unit[0] >= sp.full_units) return;
    part_kb0[0] = 0;
    part_kb1[0] = nkb;
  } else {
    const int piece = (int)blockIdx.x - full8;
    const int it0 = piece * sp.len, it1 = min(it0 + sp.len, sp.tail_units * nkb);
    if (piece >= sp.pieces || it0 >= it1) return;
    const int t0 = it0 / nkb, t1 = (it1 - 1) / nkb;
    part_unit[0] = sp.full_units + t0;
    part_kb0[0] = it0 - t0 * nkb;
    part_kb1[0] = t1 == t0 ? it1 - t0 * nkb : nkb;
    if (t1 != t0) {
      nparts = 2;
      part_unit[1] = sp.full_units + t1;
      part_kb0[1] = 0;
      part_kb1[1] = it1 - t1 * nkb;
    }
  }
  for (int part = 0; part < (SPLIT ? nparts : 1); ++part) {
  const int unit = part_unit[part];
  const int kb_begin = SPLIT ? part_kb0[part] : 0, kb_end = SPLIT ? part_kb1[part] : nkb;
  const int qblk = unit % nqb;
  const int h = (unit / nqb) % p.heads, b = unit / (nqb * p.heads);
  const int64_t q0 = (int64_t)qblk * QB + wave * 32;
  if (SPLIT && part) __syncthreads();  // the stages of the previous part have been read for the last time

  const uint16_t* qbase[2];
  const uint8_t* kbase[2];
  const uint8_t* vbase[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    qbase[s] = (const uint16_t*)p.q[s] + (int64_t)b * p.q_sb[s] + (int64_t)h * p.q_sh[s];
    kbase[s] = (const uint8_t*)((const uint16_t*)p.k[s] + (int64_t)b * p.k_sb[s] + (int64_t)h * p.k_sh[s]);
    vbase[s] = (const uint8_t*)((const uint16_t*)p.v[s] + (int64_t)b * p.v_sb[s] + (int64_t)h * p.v_sh[s]);
  }

  // ---- async K/V block loads.  One wave instruction = 1 KiB = 4 keys x 256 B; lane l lands at key
  //      l/16, physical chunk l%16.  Per block a wave issues 2 K and 2 V instructions (8 keys).
  //      Each lane keeps the global address of its 16 bytes of the block last issued; inside a
  //      segment the next block is one uniform stride further on, so the address arithmetic
  //      (clamp, segment select, 64-bit multiply) runs only for blocks that touch a segment
  //      boundary or the ragged end.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int ld_r = lane >> 4, ld_p = lane & 15;
  const uint8_t* kp[2];
  const uint8_t* vp[2];
  int ptr_seg = -1;  // segment the pointers advance in; -1: recompute
  auto set_ptrs = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = (wave * 2 + i) * 4 + ld_r;
      int64_t key = (int64_t)kb * KB + row;
      if (key >= Skv) key = Skv - 1;
      const int seg = key >= p.skv[0] ? 1 : 0;
      const int64_t lrow = key - (seg ? p.skv[0] : 0);
      kp[i] = kbase[seg] + lrow * p.k_ss[seg] * 2 + ((ld_p ^ (row & 15)) << 4);
      vp[i] = vbase[seg] + lrow * p.v_ss[seg] * 2 + ((ld_p ^ ((row & 3) << 2)) << 4);
    }
  };
  // uniform per-block pointer strides (bytes) of both segments, and the key counts as 32-bit scalars (the
  // host bounds the sequence lengths), so that the per-interval bookkeeping is a few scalar instructions
  const int skv0 = (int)p.skv[0], skv_all = (int)Skv;
  const int64_t kstep[2] = {p.k_ss[0] * (2 * KB), p.k_ss[1] * (2 * KB)};
  const int64_t vstep[2] = {p.v_ss[0] * (2 * KB), p.v_ss[1] * (2 * KB)};
  auto advance_to = [&](int kb) {  // called with consecutive kb
    const int k0 = kb * KB;
    const int lo = k0 >= skv0 ? 1 : 0, hi = k0 + KB - 1 >= skv0 ? 1 : 0;
    const bool simple = lo == hi && k0 + KB <= skv_all;
    if (__builtin_expect(simple && ptr_seg == lo, 1)) {
      const int64_t ks = lo ? kstep[1] : kstep[0], vs = lo ? vstep[1] : vstep[0];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        kp[i] += ks;
        vp[i] += vs;
      }
    } else {
      set_ptrs(kb);
    }
    ptr_seg = simple ? lo : -1;
  };
  // The async loads are written as inline assembly on purpose: for a compiler-visible LDS-DMA the
  // compiler cannot tell that the transposing LDS reads below never touch a stage that is still being
  // filled, and puts s_waitcnt vmcnt(0) in front of them, which drains the whole prefetch pipeline in
  // every interval.  Ordering against the reads is kept by hand: vmcnt waits + workgroup barriers.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)smem;
  // (M0 carries the LDS destination; nothing else in this kernel uses M0)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  auto dma16 = [&](const uint8_t* src, uint32_t lds_addr) {  // 64 lanes x 16 B -> lds_addr + lane*16
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(src), "s"(lds_addr)
                 : "memory", "m0");
  };
#pragma clang diagnostic pop
  // one 1 KiB piece of the block the pointers address: which = 0, 1 -> K rows, 2, 3 -> V rows
  auto issue_piece = [&](int stage, int which) {
    const uint32_t sK = lds0 + stage * kTile + wave_u * 2048;
    const uint32_t sV = sK + kStages * kTile;
    if (which < 2)
      dma16(kp[which], sK + which * 1024);
    else
      dma16(vp[which - 2], sV + (which - 2) * 1024);
  };
  auto issue_block = [&](int stage) {
#pragma unroll
    for (int w = 0; w < 4; ++w) issue_piece(stage, w);
  };
  advance_to(kb_begin);
  issue_block(0);
  if (kb_begin + 1 < kb_end) advance_to(kb_begin + 1);
  issue_block(1);
  if (kb_begin + 2 < kb_end) advance_to(kb_begin + 2);
  issue_block(2);

  // ---- Q fragments (B operand of S^T = K Q^T), pre-multiplied by scale*log2(e)
  const float c = p.softmax_scale * kLog2e;
  bf16x8 qf[8];
  {
    int64_t row = q0 + li;
    if (row >= Sq) row = Sq - 1;
    const int seg = row >= p.sq[0] ? 1 : 0;
    const uint16_t* src = qbase[seg] + (row - (seg ? p.sq[0] : 0)) * p.q_ss[seg];
    u32x4 raws[8];
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) raws[kc] = *reinterpret_cast<const u32x4*>(src + kc * 16 + g * 8);
    if (QPRE) {
      const uint16_t* nw = (const uint16_t*)p.q_norm_w[seg];
      const float* rope = p.rope ? p.rope + (int64_t)b * p.rope_sb + row * HD : nullptr;
      float rrms = 1.f;
      if (nw) {
        float ss = 0.f;
#pragma unroll
        for (int kc = 0; kc < 8; ++kc) ss += sumsq_chunk(raws[kc]);
        rrms = rsqrtf(pair_sum(ss) * (1.0f / HD) + p.norm_eps);
      }
#pragma unroll
      for (int kc = 0; kc < 8; ++kc)
        raws[kc] = norm_rope_chunk(raws[kc], nw != nullptr, rrms, nw ? nw + kc * 16 + g * 8 : nullptr,
                                   rope ? rope + kc * 16 + g * 8 : nullptr);
    }
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) {
      const u32x4 raw = raws[kc];
      u32x4 sc;
      sc.x = pack_bf16x2(bf16_lo(raw.x) * c, bf16_hi(raw.x) * c);
      sc.y = pack_bf16x2(bf16_lo(raw.y) * c, bf16_hi(raw.y) * c);
      sc.z = pack_bf16x2(bf16_lo(raw.z) * c, bf16_hi(raw.z) * c);
      sc.w = pack_bf16x2(bf16_lo(raw.w) * c, bf16_hi(raw.w) * c);
      qf[kc] = __builtin_bit_cast(bf16x8, sc);
    }
  }

  f32x16 oacc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_ref = 0.f;     // softmax reference of the lane's query (log2 domain)
  bool any_ref = false;  // wave-uniform: some lane of this wave has m_ref != 0
  float l_run = 0.f;

  // transposing V reads: source-lane role of this lane inside its 16-lane group
  const int grp = lane >> 4, j16 = lane & 15;
  const int tr_key = ((grp >> 1) << 2) + (j16 >> 2);    // 4*g of the receiving lanes + key within the quad
  const int tr_dbyte = (grp & 1) * 32 + (j16 & 3) * 8;  // + dt*64, bytes within the 256-byte row
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // LDS read addresses = one lane-dependent VGPR per swizzle class + an immediate: the XOR
  // swizzles only permute the 16-byte chunk (K) / 64-byte group (V) index by lane-constant bits.
  //   K fragment (kt, kc): key kt*32 + li, chunk (2kc+g) ^ (li & 15)
  //   V^T datum (key0 + 32kt + 16ch + 8hi, dt): 64-byte group dt ^ (tr_key & 3), byte tr_dbyte within
  uint32_t lane_k[8], lane_v[4];
#pragma unroll
  for (int kc = 0; kc < 8; ++kc) lane_k[kc] = li * 256 + (((2 * kc + g) ^ (li & 15)) << 4);
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
    lane_v[dt] = kStages * kTile + tr_key * 256 + ((dt ^ (tr_key & 3)) << 6) + tr_dbyte;

  // Software pipeline over 64-key blocks.  Interval kb (behind one workgroup barrier) runs
  //   stage 1:  S(kb+1)^T = K(kb+1) Q^T, 16 MFMAs;
  //   stage 2:  O^T += V(kb)^T P(kb)^T, 16 MFMAs;
  // and the softmax of the wave's own scores is spread over the 32 MFMA slots so that neither stage asks
  // more of the VALU than the matrix pipe leaves time for when two waves share a SIMD: entries
  // kExpEarly.. of P(kb) = exp2(S(kb)) in stage 1, the block maximum of S(kb+1) in the first slots of
  // stage 2 (the PV MFMAs issued there cover the latency of the last QK MFMA), entries 0..kExpEarly-1 of
  // P(kb+1) in the rest of stage 2.  The MFMAs execute while the wave issues the exp2 / convert / add
  // work on independent registers.  Without this a wave alternates MFMA-only and VALU-only phases, the
  // two waves of a SIMD do so in step (they leave the barrier together), and the matrix pipe idles
  // through every softmax.
  // Four stages of K and V: block kb+1 must have landed when interval kb starts, kb+2 is in flight,
  // kb+3 is issued into the stage block kb-1 has left.
  constexpr int kExpEarly = 12;  // even; entries of P(kb+1) produced during stage 2 of interval kb
  constexpr int kAhead = 2;      // operand fragments in flight ahead of the MFMA that uses them
  auto interval_head = [&](int kb) {
    __builtin_amdgcn_s_waitcnt(0x0f74);  // vmcnt(4): only block kb+2 may still be in flight
    __builtin_amdgcn_s_barrier();
    if (__builtin_expect(kb + 3 < kb_end, 1)) advance_to(kb + 3);  // else: re-fetch the last block, nobody reads it
  };
  // Softmax reference.  mask_tail masks the ragged tail of block `blk`; ref_scan subtracts the current
  // reference and returns the block maximum of the lane's query; ref_move shifts the reference (rescaling O and l), which
  // is needed only when a block maximum leaves the safe range.
  auto mask_tail = [&](f32x16 (&s)[2], int blk) {
    if (__builtin_expect((blk + 1) * KB > skv_all, 0)) {  // ragged tail of the key axis
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = blk * KB + kt * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
          if (key >= skv_all) s[kt][r] = -INFINITY;
        }
    }
  };
  auto ref_scan = [&](f32x16 (&s)[2], int blk) -> float {
    if (__builtin_expect(any_ref, 0)) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[kt][r] -= m_ref;
    }
    float m0 = max3(s[0][0], s[0][1], s[0][2]);
    float m1 = max3(s[1][0], s[1][1], s[1][2]);
#pragma unroll
    for (int r = 3; r < 15; r += 2) {
      m0 = max3(m0, s[0][r], s[0][r + 1]);
      m1 = max3(m1, s[1][r], s[1][r + 1]);
    }
    return pair_max(max3(m0, m1, fmaxf(s[0][15], s[1][15])));
  };
  auto ref_must_move = [&](float mx, int blk) -> bool {  // wave-uniform
    const bool move = mx > kRescaleThreshold || (blk == kb_begin && mx < -kRescaleThreshold);
    return __builtin_amdgcn_ballot_w64(move) != 0;
  };
  auto ref_move = [&](f32x16 (&s)[2], float mx, int blk) -> float {
    any_ref = true;
    const float d = blk == kb_begin ? mx : fmaxf(mx, 0.f);
    const float alpha = blk == kb_begin ? 1.0f : __builtin_amdgcn_exp2f(-d);
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kt][r] -= d;
    m_ref += d;
    l_run *= alpha;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
    return alpha;
  };
  // entry e (0..31) of P = exp2(S'): score s[e/16][e%16]; two entries pack into one bf16x2 word of the PV
  // operand.  The row sum adds the fp32 values with plain v_add_f32 (v_dot2c_f32_bf16 on the packed pair
  // would be one instruction, but it executes on the matrix pipe and was measured to cost a third of the
  // MFMA rate).
  // Each result is pinned where it is computed by an empty volatile asm that "uses" it: the exponential, the
  // convert and the add are pure, and the optimiser otherwise sinks them to the block of their first use (the
  // PV MFMAs behind the next branch, the row sum at the end of the interval), past the scheduling barriers:
  // the MFMA slots they were written into then run bare and the VALU work runs in MFMA-free clumps.
  float p_even = 0.f, lsum0 = 0.f, lsum1 = 0.f;
  auto exp_entry = [&](const f32x16 (&s)[2], uint32_t (&pw)[2][8], int e) {
    float pv = __builtin_amdgcn_exp2f(s[e >> 4][e & 15]);
    if (e & 1) {
      uint32_t w = pack_bf16x2(p_even, pv);
      lsum1 += pv;
      asm volatile("" : "+v"(w), "+v"(lsum1));
      pw[e >> 4][(e & 15) >> 1] = w;
    } else {
      lsum0 += pv;
      asm volatile("" : "+v"(pv), "+v"(lsum0));
      p_even = pv;
    }
  };
  auto qk = [&](f32x16 (&s)[2], int stage) {
    const uint8_t* sK = smem + stage * kTile;
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(sK + lane_k[kc] + kt * 8192);
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kc], kc == 0 ? zero16 : s[kt], 0, 0, 0);
      }
    }
  };
  typedef short v8i16 __attribute__((ext_vector_type(8)));
  // one interval; `stage` (= kb % 4) is a literal so that every LDS offset folds into an immediate.
  // pw_cur holds entries 0..kExpEarly-1 of P(kb) on entry; pw_next holds those of P(kb+1) on exit.
  auto interval = [&](int kb, int stage, f32x16 (&s_cur)[2], f32x16 (&s_next)[2], uint32_t (&pw_cur)[2][8],
                      uint32_t (&pw_next)[2][8]) {
    interval_head(kb);
    // The next block's four 1 KiB pieces go out between the MFMAs, K in stage 1 and V in stage 2: the CU's
    // one address path takes ~25 cycles per piece, and a wave whose load queues behind the other waves'
    // loads cannot issue its MFMAs meanwhile (32 pieces at once right after the barrier cost every wave
    // 500-800 cycles).
    constexpr int kLoadSlots[4] = {3, 11, 7, 13};
    // ---- stage 1: 16 slots, each = [LDS read of the K fragment two MFMAs ahead, one MFMA of S(kb+1),
    //      one or two entries of P(kb)]; sched_barrier pins the order
    const uint8_t* sK = smem + ((stage + 1) % kStages) * kTile;
    auto k_frag = [&](int i) {  // MFMA i of the block: k-chunk i/2, key tile i%2
      return *reinterpret_cast<const bf16x8*>(sK + lane_k[i >> 1] + (i & 1) * 8192);
    };
    const uint8_t* sV = smem + stage * kTile;  // lane_v carries the offset of the V region
    auto v_frag = [&](int j) {  // MFMA j: 16-key chunk j/4 (kt = j/8, ch = (j/4)%2), d tile j%4
      const uint8_t* src = sV + lane_v[j & 3] + (j >> 2) * 16 * 256;
      const v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4i16*)src);
      const v4i16 hi =
          __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4i16*)(src + 8 * 256));
      const v8i16 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      return __builtin_bit_cast(bf16x8, both);
    };
    // operand fragments are read kAhead MFMAs before their use; the last slots of stage 1 already fetch
    // the first V^T fragments of stage 2 (block kb landed long ago), so only stage 1 starts cold
    constexpr int kLate = 32 - kExpEarly;  // entries left for stage 1; the first kLate-16 slots take two
    bf16x8 kf[kAhead + 1], vf[kAhead + 1];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) kf[i] = k_frag(i);
    int e = kExpEarly;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (i + kAhead < 16)
        kf[(i + kAhead) % (kAhead + 1)] = k_frag(i + kAhead);
      else
        vf[(i + kAhead - 16) % (kAhead + 1)] = v_frag(i + kAhead - 16);
      const int kt = i & 1;
      s_next[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % (kAhead + 1)], qf[i >> 1], i < 2 ? zero16 : s_next[kt], 0, 0, 0);
      exp_entry(s_cur, pw_cur, e++);
      if (i < kLate - 16) exp_entry(s_cur, pw_cur, e++);
      if (i == kLoadSlots[0]) issue_piece((stage + 3) % kStages, 0);
      if (i == kLoadSlots[1]) issue_piece((stage + 3) % kStages, 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    l_run += lsum0 + lsum1;
    lsum0 = lsum1 = 0.f;
    // ---- stage 2: O^T += V^T P^T, 16 slots = [transposing LDS reads of a V^T operand, one MFMA].
    //      16-key chunk (kt, ch): slots 8g..8g+7 = keys {4g..4g+3, 8+4g..8+4g+3}
    auto pv_slot = [&](int j) {
      if (j + kAhead < 16) vf[(j + kAhead) % (kAhead + 1)] = v_frag(j + kAhead);
      const int kt = j >> 3, ch = (j >> 2) & 1, dt = j & 3;
      const u32x4 w = {pw_cur[kt][4 * ch + 0], pw_cur[kt][4 * ch + 1], pw_cur[kt][4 * ch + 2], pw_cur[kt][4 * ch + 3]};
      oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[j % (kAhead + 1)], __builtin_bit_cast(bf16x8, w), oacc[dt], 0, 0, 0);
    };
    constexpr int kScanSlots = 4;  // PV MFMAs issued before the block maximum of S(kb+1) is looked at
#pragma unroll
    for (int j = 0; j < kScanSlots; ++j) {
      pv_slot(j);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (__builtin_expect(kb + 1 < kb_end, 1)) {
      mask_tail(s_next, kb + 1);
      const float mx = SCAN ? ref_scan(s_next, kb + 1) : 0.f;
      if (SCAN && __builtin_expect(ref_must_move(mx, kb + 1), 0)) {
        // rare: O, l and the scores of block kb+1 move to the new reference now; the part of P(kb) that
        // the remaining PV MFMAs still have to accumulate follows (one more bf16 rounding on it)
        const float alpha = ref_move(s_next, mx, kb + 1);
#pragma unroll
        for (int j = kScanSlots; j < 16; j += 4)
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            uint32_t& word = pw_cur[j >> 3][4 * ((j >> 2) & 1) + w];
            word = pack_bf16x2(bf16_lo(word) * alpha, bf16_hi(word) * alpha);
          }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // (in the last interval the entries below come from a block that does not exist and are dropped)
    int e2 = 0;
#pragma unroll
    for (int j = kScanSlots; j < 16; ++j) {
      pv_slot(j);
      // kExpEarly entries over the 16 - kScanSlots remaining slots, the surplus in the first ones
      exp_entry(s_next, pw_next, e2++);
      if (j - kScanSlots < kExpEarly - (16 - kScanSlots)) exp_entry(s_next, pw_next, e2++);
      if (j == kLoadSlots[2]) issue_piece((stage + 3) % kStages, 2);
      if (j == kLoadSlots[3]) issue_piece((stage + 3) % kStages, 3);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  f32x16 sA[2], sB[2];
  uint32_t pwA[2][8], pwB[2][8];
  __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8): block 0 has landed
  __builtin_amdgcn_s_barrier();
  qk(sA, 0);
  {
    mask_tail(sA, kb_begin);
    if (SCAN) {
      const float mx = ref_scan(sA, kb_begin);
      if (ref_must_move(mx, kb_begin)) ref_move(sA, mx, kb_begin);
    }
#pragma unroll
    for (int e = 0; e < kExpEarly; ++e) exp_entry(sA, pwA, e);
  }
  for (int kb = kb_begin; kb < kb_end; kb += 4) {  // stage of block kb = (kb - kb_begin) % 4
    interval(kb, 0, sA, sB, pwA, pwB);
    if (kb + 1 < kb_end) interval(kb + 1, 1, sB, sA, pwB, pwA);
    if (kb + 2 < kb_end) interval(kb + 2, 2, sA, sB, pwA, pwB);
    if (kb + 3 < kb_end) interval(kb + 3, 3, sB, sA, pwB, pwA);
  }
  __builtin_amdgcn_s_waitcnt(0);  // drain trailing async loads

  // ---- lane (g, j): query j, d = dt*32 + 8*(r/4) + 4g + r%4
  const float l_row = pair_sum(l_run);
  const int64_t row = q0 + li;
  if (!SPLIT || (kb_begin == 0 && kb_end == nkb)) {  // the whole key axis: normalise and store
    if (row < Sq) store_output(p, b, h, row, g, oacc, 1.0f / l_row);
  } else {                               // a part: leave O, l and the reference for the merge
    const int t = unit - sp.full_units;
    const int first_piece = (t * nkb) / sp.len;
    const int my_piece = (t * nkb + kb_begin) / sp.len;
    float* slot = sp.slots + (int64_t)(t * sp.max_parts + (my_piece - first_piece)) * kSlotFloats;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const f32x4 v = {oacc[dt][4 * rq + 0], oacc[dt][4 * rq + 1], oacc[dt][4 * rq + 2], oacc[dt][4 * rq + 3]};
        *reinterpret_cast<f32x4*>(slot + ((((dt * 4 + rq) * 8 + wave) * 2 + g) * 32 + li) * 4) = v;
      }
    if (g == 0) {
      slot[kSlotOFloats + wave * 32 + li] = l_row;
      slot[kSlotOFloats + QB + wave * 32 + li] = m_ref;
    }
  }
  }  // parts
}

// Combines the parts of every split unit: O = sum_i O_i 2^(m_i - m), l likewise, m = max_i m_i.
// Same lane <-> (query, d) mapping as the attention kernel, so the slots are read as they were written.
// blockIdx.y picks one of the sixteen (dt, rq) groups of four output columns: a unit's merge is spread over
// sixteen workgroups, each reading one 16-byte vector per lane and part (a unit cut into many parts would
// otherwise be read, 128 KiB per part, by a single workgroup).
__global__ __launch_bounds__(512) void attn_merge_kernel(dsx_attn_params p, AttnSplit sp) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 5, li = lane & 31;
  const int nqb = (int)((p.sq[0] + p.sq[1] + QB - 1) / QB);
  const int64_t Sq = p.sq[0] + p.sq[1];
  const int nkb = (int)((p.skv[0] + p.skv[1] + KB - 1) / KB);
  const int t = blockIdx.x;
  const int dt = (int)blockIdx.y >> 2, rq = (int)blockIdx.y & 3;
  const int first_piece = (t * nkb) / sp.len, last_piece = ((t + 1) * nkb - 1) / sp.len;
  const int np = last_piece - first_piece + 1;
  if (np == 1) return;  // the unit was covered by one piece, which wrote the output itself
  const int unit = sp.full_units + t;
  const int qblk = unit % nqb;
  const int h = (unit / nqb) % p.heads, b = unit / (nqb * p.heads);
  const float* base = sp.slots + (int64_t)t * sp.max_parts * kSlotFloats;
  const int qi = wave * 32 + li;
  float m = -INFINITY;
  for (int i = 0; i < np; ++i) m = fmaxf(m, base[(int64_t)i * kSlotFloats + kSlotOFloats + QB + qi]);
  f32x4 o = {0.f, 0.f, 0.f, 0.f};
  float l = 0.f;
  for (int i = 0; i < np; ++i) {
    const float* slot = base + (int64_t)i * kSlotFloats;
    const float w = __builtin_amdgcn_exp2f(slot[kSlotOFloats + QB + qi] - m);
    l += slot[kSlotOFloats + qi] * w;
    const f32x4 v = *reinterpret_cast<const f32x4*>(slot + ((((dt * 4 + rq) * 8 + wave) * 2 + g) * 32 + li) * 4);
#pragma unroll
    for (int c = 0; c < 4; ++c) o[c] += v[c] * w;
  }
  const int64_t row = (int64_t)qblk * QB + qi;
  if (row >= Sq) return;
  const float inv = 1.0f / l;
  const int seg = row >= p.sq[0] ? 1 : 0;
  uint16_t* dst = (uint16_t*)p.o[seg] + (int64_t)b * p.o_sb[seg] + (int64_t)h * p.o_sh[seg] +
                  (row - (seg ? p.sq[0] : 0)) * p.o_ss[seg];
  u32x2 w2;
  w2.x = pack_bf16x2(o[0] * inv, o[1] * inv);
  w2.y = pack_bf16x2(o[2] * inv, o[3] * inv);
  *reinterpret_cast<u32x2*>(dst + dt * 32 + 8 * rq + 4 * g) = w2;
}

}  // namespace

// Decides whether the last round of workgroups is worth splitting along the keys and lays the split out.
// `cus` compute units, U units of nkb key blocks.  Returns the scratch bytes the split needs (0: no split).
static int64_t plan_split(const dsx_attn_params& p, int cus, AttnSplit& sp) {
  const int64_t Sq = p.sq[0] + p.sq[1], Skv = p.skv[0] + p.skv[1];
  const int64_t units = ((Sq + QB - 1) / QB) * p.heads * p.batch;
  const int nkb = (int)((Skv + KB - 1) / KB);
  sp = AttnSplit{(int)units, 0, 0, 1, 1, nullptr, 0};
  if (p.rope || p.q_norm_w[0] || p.q_norm_w[1]) return 0;  // the split kernel has no q pre-processing
  if (cus <= 0) return 0;                                    // no device to ask
  const int tail = (int)(units % cus);
  const int64_t rounds = (units + cus - 1) / cus;
  // Worth it when the compute units left idle in the last round are at least a quarter of the whole launch
  // and the key axis is long enough for the parts to dwarf the cost of writing and merging them (~20 us).
  // Below that the split loses: the chip is power-limited during attention, so a last round on fewer
  // compute units runs at a higher clock (measured at 432 units on 256 compute units: 252 us whole,
  // 265 us split; at 384 units: 218 us whole, 207 us split).
  if (tail == 0 || nkb < 32 || (int64_t)(cus - tail) * 4 < rounds * cus) return 0;
  // One piece per compute unit, but no more than eight per unit: every piece leaves 130 KiB of partial results
  // that the merge reads back, and a handful of units cut into 256 slivers costs more there than it saves here.
  const int pieces = (int)std::min<int64_t>(cus, (int64_t)tail * 8);
  const int len = (int)(((int64_t)tail * nkb + pieces - 1) / pieces);
  // What the split saves against what it costs, from measurements on this chip: a 64-key block of a workgroup
  // takes ~1.65 us; a part (a piece, or the piece's share of a second unit) costs ~0.09 us of writing and reading
  // back its 130 KiB, the merge launch ~8 us.  (2048 x 2048 x 24 heads = 192 units: 59 us whole, 85 us cut into
  // 256 pieces of 24 blocks; 2816 x 2816 = 264 units: 144 us whole, 114 us with its last 8 units cut into 64.)
  const double saved_us = (nkb - len) * 1.65, cost_us = (pieces + tail) * 0.09 + 8.0;
  if (saved_us < 1.25 * cost_us) return 0;
  sp.full_units = (int)(units - tail);
  sp.tail_units = tail;
  sp.pieces = pieces;
  sp.len = len;
  sp.max_parts = (nkb + sp.len - 1) / sp.len + 1;
  return (int64_t)tail * sp.max_parts * kSlotFloats * (int64_t)sizeof(float);
}

int64_t attn_plain_workspace_bytes(const dsx_attn_params& p) {
  AttnSplit sp;
  return plan_split(p, device_cus(), sp);
}

// `scratch` / `scratch_bytes`: optional device memory for the key-range split (may be null).
int launch_attn_plain(const dsx_attn_params& p, void* scratch, int64_t scratch_bytes, hipStream_t st) {
  static PerDeviceOnce attr_once;
  const int attr_rc = per_device_once(attr_once, [](int) {
    const void* kernels[6] = {
        (const void*)attn_plain_kernel<true, true, false>,   (const void*)attn_plain_kernel<false, true, false>,
        (const void*)attn_plain_kernel<true, false, false>,  (const void*)attn_plain_kernel<false, false, false>,
        (const void*)attn_plain_kernel<true, false, true>,   (const void*)attn_plain_kernel<false, false, true>};
    for (const void* kfn : kernels)
      if (hipFuncSetAttribute(kfn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess)
        return (int)DSX_ELAUNCH;
    return (int)DSX_OK;
  });
  if (attr_rc != DSX_OK) return attr_rc;
  const int64_t Sq = p.sq[0] + p.sq[1];
  const int64_t units = ((Sq + QB - 1) / QB) * p.heads * p.batch;
  if (units > (1ll << 30)) return DSX_EBADSHAPE;
  // Three full rounds of workgroups and more run into the chip's power limit, where the 16x16x32 form of the kernel
  // is the faster one (attn_plain16.hip); below that this one is.
  const int cus = device_cus();
  const bool qpre_any = p.rope || p.q_norm_w[0] || p.q_norm_w[1];
  if (cus > 0 && units >= 3 * (int64_t)cus && !qpre_any) return launch_attn_plain16(p, units, st);
  AttnSplit sp;
  const int64_t need = plan_split(p, cus, sp);
  if (need == 0 || !scratch || scratch_bytes < need || ((uintptr_t)scratch & 15))
    sp = AttnSplit{(int)units, 0, 0, 1, 1, nullptr, 0};
  else
    sp.slots = (float*)scratch;
  dim3 grid((unsigned)(((sp.full_units + 7) / 8) * 8 + sp.pieces)), block(512);
  // a caller-supplied bound on |softmax_scale * q.k| that keeps exp2 of every score inside fp32 and bf16
  // with a fixed reference lets the kernel skip the per-block maximum
  const bool bounded = p.score_bound > 0.f && p.score_bound * kLog2e <= kRescaleThreshold;
  const bool split = sp.tail_units > 0;
  const bool qpre = p.rope || p.q_norm_w[0] || p.q_norm_w[1];  // (never together with the split)
  sp.device_bound = 0;
  if (p.qk_norm2_max && !bounded && !qpre) {
    // the bound lives on the device: launch both variants, each looks at it and one of them returns at once
    sp.device_bound = 1;
    if (split) {
      attn_plain_kernel<false, true, false><<<grid, block, kLdsBytes, st>>>(p, sp);
      attn_plain_kernel<true, true, false><<<grid, block, kLdsBytes, st>>>(p, sp);
    } else {
      attn_plain_kernel<false, false, false><<<grid, block, kLdsBytes, st>>>(p, sp);
      attn_plain_kernel<true, false, false><<<grid, block, kLdsBytes, st>>>(p, sp);
    }
  } else if (qpre && bounded)
    attn_plain_kernel<false, false, true><<<grid, block, kLdsBytes, st>>>(p, sp);
  else if (qpre)
    attn_plain_kernel<true, false, true><<<grid, block, kLdsBytes, st>>>(p, sp);
  else if (bounded && split)
    attn_plain_kernel<false, true, false><<<grid, block, kLdsBytes, st>>>(p, sp);
  else if (bounded)
    attn_plain_kernel<false, false, false><<<grid, block, kLdsBytes, st>>>(p, sp);
  else if (split)
    attn_plain_kernel<true, true, false><<<grid, block, kLdsBytes, st>>>(p, sp);
  else
    attn_plain_kernel<true, false, false><<<grid, block, kLdsBytes, st>>>(p, sp);
  if (hipGetLastError() != hipSuccess) return DSX_ELAUNCH;
  if (sp.tail_units > 0) {
    attn_merge_kernel<<<dim3((unsigned)sp.tail_units, 16), block, 0, st>>>(p, sp);
    if (hipGetLastError() != hipSuccess) return DSX_ELAUNCH;
  }
  return DSX_OK;
}

}  // namespace dsx
