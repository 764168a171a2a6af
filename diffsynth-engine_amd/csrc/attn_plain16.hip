// Flash attention forward for gfx950, the form for launches of many full rounds of workgroups (q and k already
// normalised and rotated): head dim 128, bf16 operands, fp32 online softmax.  Same work split, LDS staging and
// softmax as attn_plain.hip; what differs is the MFMA shape and with it every register layout.  Under the power
// limit, which a launch that keeps every compute unit busy for several rounds runs into, this shape draws less per
// flop (28 heads x 9216 tokens: 922 against 958 us); where compute units idle and the clock is not limited it
// issues twice as many MFMAs beside the same softmax work and is the slower one (8 heads x 4608 tokens: 109
// against 98 us), so launch_attn_plain picks by the number of rounds.
//
// MFMA formulation: S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_16x16x32_bf16 (on N(0,1) operands, where the chip
// runs at its power limit, a bare stream of this shape sustains 12 % more than one of v_mfma_f32_32x32x16_bf16:
// 2.08 against 1.86 PFLOP/s).  A wave owns 32 queries = two 16-query MFMA columns; lane (q = lane / 16,
// i = lane % 16) holds, for each of its two queries 16t + i, the scores of keys 16kt + 4q .. 4q + 3 of every
// 16-key tile kt: a query's row is spread over the four lanes i, i + 16, i + 32, i + 48, so the exponentials are
// lane-local and only row maxima / row sums cross lanes (two permlane swaps).  Packed to bf16, the scores of two
// neighbouring key tiles are exactly the B operand of the second product (K extent 32 keys): no LDS round trip.
//
// Work split: one workgroup = 8 waves = 256 consecutive queries of one (batch, head); every wave needs ~240 VGPRs,
// so two waves share a SIMD and one workgroup fills a CU.  While one wave of a SIMD works through
// exp2/convert/row-sum on the VALU, the other's MFMAs can keep the matrix pipe busy.
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
// LDS swizzles: K rows (256 B): 16-byte chunk c of key r at c ^ (r & 15)        (ds_read_b128 by 16 rows x 4 chunks);
//               V rows (256 B): chunk c of key r at c ^ ((r & 7) << 1)          (transposing 8-byte reads of
//                                                                                16 keys x 32 bytes).
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

// Reductions over the four lanes i, i + 16, i + 32, i + 48 that share a query.  permlane16_swap(v, v) returns
// (rows 0 0 2 2, rows 1 1 3 3) of v, permlane32_swap(v, v) (lower half twice, upper half twice).
__device__ __forceinline__ float quad_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  const float m = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(m), __float_as_uint(m), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  const float m = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(m), __float_as_uint(m), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

// normalised output of one lane for one of its two queries: query `row`, d = dt*16 + 4q + 0..3 per dt
__device__ __forceinline__ void store_output(const dsx_attn_params& p, int b, int h, int64_t row, int q4,
                                             const f32x4 (&oacc)[8][2], int t, float inv) {
  const int seg = row >= p.sq[0] ? 1 : 0;
  uint16_t* dst = (uint16_t*)p.o[seg] + (int64_t)b * p.o_sb[seg] + (int64_t)h * p.o_sh[seg] +
                  (row - (seg ? p.sq[0] : 0)) * p.o_ss[seg];
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) {
    u32x2 w;
    w.x = pack_bf16x2(oacc[dt][t][0] * inv, oacc[dt][t][1] * inv);
    w.y = pack_bf16x2(oacc[dt][t][2] * inv, oacc[dt][t][3] * inv);
    *reinterpret_cast<u32x2*>(dst + dt * 16 + 4 * q4) = w;
  }
}

// SCAN = false: the caller has bounded every |score| (log2 domain) by kRescaleThreshold, so the softmax
// reference can stay 0 for the whole row and the per-block maximum is not computed at all.
// device_bound: both variants were launched and the two floats behind p.qk_norm2_max say which one works.
template <bool SCAN>
__global__ __launch_bounds__(512) void attn_plain16_kernel(dsx_attn_params p, int units, int device_bound) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  if (device_bound) {
    // Both variants were launched; the two device floats say which one works.  Not bounded (Inf and NaN
    // included, for which the comparison is false) means the variant with the running maximum.
    const float a = p.qk_norm2_max[0], b = p.qk_norm2_max[1];
    const bool bounded = sqrtf(a) * sqrtf(b) * p.softmax_scale * (kLog2e * 1.02f) <= kRescaleThreshold;
    if (bounded == SCAN) return;
  }
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;  // 0..7
  const int q4 = lane >> 4, i16 = lane & 15;
  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of (batch, head,
  // query block) units so that the query blocks of one head share that head's K/V through ONE L2
  // (with a plain 3-D grid every XCD ends up fetching every head's K and V).
  const int nqb = (int)((p.sq[0] + p.sq[1] + QB - 1) / QB);
  const int64_t Sq = p.sq[0] + p.sq[1];
  const int64_t Skv = p.skv[0] + p.skv[1];
  const int nkb = (int)((Skv + KB - 1) / KB);
  const int units8 = (units + 7) & ~7;
  const int unit = (int)(blockIdx.x & 7) * (units8 >> 3) + (int)(blockIdx.x >> 3);
  if (unit >= units) return;
  const int kb_begin = 0, kb_end = nkb;
  const int qblk = unit % nqb;
  const int h = (unit / nqb) % p.heads, b = unit / (nqb * p.heads);
  const int64_t q0 = (int64_t)qblk * QB + wave * 32;

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
      vp[i] = vbase[seg] + lrow * p.v_ss[seg] * 2 + ((ld_p ^ ((row & 7) << 1)) << 4);
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

  // ---- Q fragments (B operand of S^T = K Q^T), pre-multiplied by scale*log2(e): qf[t][dc] = query 16t + i,
  //      d = 32dc + 8q .. + 7
  const float c = p.softmax_scale * kLog2e;
  bf16x8 qf[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    int64_t row = q0 + t * 16 + i16;
    if (row >= Sq) row = Sq - 1;
    const int seg = row >= p.sq[0] ? 1 : 0;
    const uint16_t* src = qbase[seg] + (row - (seg ? p.sq[0] : 0)) * p.q_ss[seg];
    u32x4 raws[4];
#pragma unroll
    for (int dc = 0; dc < 4; ++dc) raws[dc] = *reinterpret_cast<const u32x4*>(src + dc * 32 + q4 * 8);
#pragma unroll
    for (int dc = 0; dc < 4; ++dc) {
      const u32x4 raw = raws[dc];
      u32x4 sc;
      sc.x = pack_bf16x2(bf16_lo(raw.x) * c, bf16_hi(raw.x) * c);
      sc.y = pack_bf16x2(bf16_lo(raw.y) * c, bf16_hi(raw.y) * c);
      sc.z = pack_bf16x2(bf16_lo(raw.z) * c, bf16_hi(raw.z) * c);
      sc.w = pack_bf16x2(bf16_lo(raw.w) * c, bf16_hi(raw.w) * c);
      qf[t][dc] = __builtin_bit_cast(bf16x8, sc);
    }
  }

  f32x4 oacc[8][2];  // [d tile][query column]: lane (q, i): query 16t + i, d = 16dt + 4q .. + 3
#pragma unroll
  for (int dt = 0; dt < 8; ++dt)
#pragma unroll
    for (int t = 0; t < 2; ++t) oacc[dt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_ref[2] = {0.f, 0.f};  // softmax reference of the lane's two queries (log2 domain)
  bool any_ref = false;         // wave-uniform: some lane of this wave has a reference != 0
  float l_run[2] = {0.f, 0.f};

  // transposing V reads: a 16-lane group q fetches keys 4q .. 4q + 3 of a 16-key half x 16 d; source lane j
  // of the group points at key 4q + j/4, d bytes 8 (j % 4) of the 32-byte piece of d tile dt
  const int tr_key = 4 * q4 + (i16 >> 2);
  const int tr_dbyte = (i16 & 3) * 8;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

  // LDS read addresses = one lane-dependent VGPR per swizzle class + an immediate: the XOR
  // swizzles only permute the 16-byte chunk (K) / 32-byte piece (V) index by lane-constant bits.
  //   K fragment (kt, dc): key 16kt + i, chunk (4dc + q) ^ i
  //   V^T datum (key 32c + 16hi + tr_key, dt): 32-byte piece dt ^ (tr_key & 7), byte tr_dbyte within
  uint32_t lane_k[4], lane_v[8];
#pragma unroll
  for (int dc = 0; dc < 4; ++dc) lane_k[dc] = i16 * 256 + (((4 * dc + q4) ^ i16) << 4);
#pragma unroll
  for (int dt = 0; dt < 8; ++dt)
    lane_v[dt] = kStages * kTile + tr_key * 256 + ((dt ^ (tr_key & 7)) << 5) + tr_dbyte;

  // Software pipeline over 64-key blocks.  Interval kb (behind one workgroup barrier) runs
  //   stage 1:  S(kb+1)^T = K(kb+1) Q^T, 32 MFMAs;
  //   stage 2:  O^T += V(kb)^T P(kb)^T, 32 MFMAs;
  // and the softmax of the wave's own scores is spread over the 64 MFMA slots so that neither stage asks
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
  constexpr int kAhead = 2;      // operand fragments in flight ahead of the MFMA pair that uses them
  auto interval_head = [&](int kb) {
    __builtin_amdgcn_s_waitcnt(0x0f74);  // vmcnt(4): only block kb+2 may still be in flight
    __builtin_amdgcn_s_barrier();
    if (__builtin_expect(kb + 3 < kb_end, 1)) advance_to(kb + 3);  // else: re-fetch the last block, nobody reads it
  };
  // Scores of one block: s[kt][t][e] = query 16t + i against key 16kt + 4q + e.
  // mask_tail masks the ragged tail of block `blk`; ref_scan subtracts the current reference and returns, for each of
  // the lane's two queries, the maximum over the lane's own keys; ref_move shifts the references (rescaling O and l), which is needed only when
  // a block maximum leaves the safe range.
  auto mask_tail = [&](f32x4 (&s)[4][2], int blk) {
    if (__builtin_expect((blk + 1) * KB > skv_all, 0)) {  // ragged tail of the key axis
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = blk * KB + kt * 16 + 4 * q4 + e;
          if (key >= skv_all) s[kt][0][e] = s[kt][1][e] = -INFINITY;
        }
    }
  };
  auto ref_scan = [&](f32x4 (&s)[4][2], float (&mx)[2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (__builtin_expect(any_ref, 0)) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int e = 0; e < 4; ++e) s[kt][t][e] -= m_ref[t];
      }
      float m0 = max3(s[0][t][0], s[0][t][1], s[0][t][2]);
      float m1 = max3(s[1][t][0], s[1][t][1], s[1][t][2]);
      m0 = max3(m0, s[0][t][3], s[2][t][0]);
      m1 = max3(m1, s[1][t][3], s[3][t][0]);
      m0 = max3(m0, s[2][t][1], s[2][t][2]);
      m1 = max3(m1, s[3][t][1], s[3][t][2]);
      mx[t] = max3(m0, m1, fmaxf(s[2][t][3], s[3][t][3]));  // of the lane's own 16 keys: a quarter of the row
    }
  };
  // Whether any reference of the wave has to move (wave-uniform).  Looks at the lanes' partial maxima only: a row
  // maximum above the threshold shows in one of its four lanes, and a row maximum below minus the threshold
  // shows in all four, so "some lane below" can only fire early, never late -- the move itself works with the
  // true row maxima and is harmless when it was not strictly needed.
  auto ref_must_move = [&](const float (&mx)[2], int blk) -> bool {
    const float hi = fmaxf(mx[0], mx[1]), lo = fminf(mx[0], mx[1]);
    const bool move = hi > kRescaleThreshold || (blk == kb_begin && lo < -kRescaleThreshold);
    return __builtin_amdgcn_ballot_w64(move) != 0;
  };
  auto ref_move = [&](f32x4 (&s)[4][2], const float (&part)[2], int blk, float (&alpha)[2]) {
    any_ref = true;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float mxt = quad_max(part[t]);  // the row maximum: over the four lanes that share the query
      const float d = blk == kb_begin ? mxt : fmaxf(mxt, 0.f);
      alpha[t] = blk == kb_begin ? 1.0f : __builtin_amdgcn_exp2f(-d);
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) s[kt][t][e] -= d;
      m_ref[t] += d;
      l_run[t] *= alpha[t];
#pragma unroll
      for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int e = 0; e < 4; ++e) oacc[dt][t][e] *= alpha[t];
    }
  };
  // Entry n (0..31) of P = exp2(S'), in the order the second product consumes them: 32-key chunk n / 16, query
  // column (n / 8) % 2, word (n / 2) % 4 of that column's B operand -- words 0, 1 hold keys 4q .. 4q + 3 of the
  // chunk's first key tile, words 2, 3 those of its second -- low or high half n % 2.  The row sum adds the fp32
  // values with plain v_add_f32 (v_dot2c_f32_bf16 on the packed pair would be one instruction, but it executes
  // on the matrix pipe and was measured to cost a third of the MFMA rate).
  // Each result is pinned where it is computed by an empty volatile asm that "uses" it: the exponential, the
  // convert and the add are pure, and the optimiser otherwise sinks them to the block of their first use (the
  // PV MFMAs behind the next branch, the row sum at the end of the interval), past the scheduling barriers:
  // the MFMA slots they were written into then run bare and the VALU work runs in MFMA-free clumps.
  float p_even = 0.f, lsum[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
  auto exp_entry = [&](const f32x4 (&s)[4][2], uint32_t (&pw)[2][2][4], int n) {
    const int ch = n >> 4, t = (n >> 3) & 1, w = (n >> 1) & 3;
    float pv = __builtin_amdgcn_exp2f(s[2 * ch + (w >> 1)][t][2 * (w & 1) + (n & 1)]);
    if (n & 1) {
      uint32_t word = pack_bf16x2(p_even, pv);
      lsum[t][1] += pv;
      asm volatile("" : "+v"(word), "+v"(lsum[t][1]));
      pw[ch][t][w] = word;
    } else {
      lsum[t][0] += pv;
      asm volatile("" : "+v"(pv), "+v"(lsum[t][0]));
      p_even = pv;
    }
  };
  // first block: S(0) with nothing to overlap
  auto qk = [&](f32x4 (&s)[4][2], int stage) {
    const uint8_t* sK = smem + stage * kTile;
#pragma unroll
    for (int dc = 0; dc < 4; ++dc)
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(sK + lane_k[dc] + kt * 4096);
#pragma unroll
        for (int t = 0; t < 2; ++t)
          s[kt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[t][dc], dc == 0 ? zero4 : s[kt][t], 0, 0, 0);
      }
  };
  typedef short v8i16 __attribute__((ext_vector_type(8)));
  // one interval; `stage` (= kb % 4) is a literal so that every LDS offset folds into an immediate.
  // pw_cur holds entries 0..kExpEarly-1 of P(kb) on entry; pw_next holds those of P(kb+1) on exit.
  auto interval = [&](int kb, int stage, f32x4 (&s_cur)[4][2], f32x4 (&s_next)[4][2], uint32_t (&pw_cur)[2][2][4],
                      uint32_t (&pw_next)[2][2][4]) {
    interval_head(kb);
    // The next block's four 1 KiB pieces go out between the MFMAs, K in stage 1 and V in stage 2: the CU's
    // one address path takes ~25 cycles per piece, and a wave whose load queues behind the other waves'
    // loads cannot issue its MFMAs meanwhile (32 pieces at once right after the barrier cost every wave
    // 500-800 cycles).
    constexpr int kLoadSlots[4] = {3, 11, 7, 13};  // in operand fragments (= MFMA pairs)
    // ---- stage 1: 16 operand fragments, each = [LDS read of the K fragment two fragments ahead, two MFMAs of
    //      S(kb+1) (the two query columns), entries of P(kb)]; sched_barrier pins the order
    const uint8_t* sK = smem + ((stage + 1) % kStages) * kTile;
    auto k_frag = [&](int f) {  // fragment f of the block: d chunk f/4, key tile f%4
      return *reinterpret_cast<const bf16x8*>(sK + lane_k[f >> 2] + (f & 3) * 4096);
    };
    const uint8_t* sV = smem + stage * kTile;  // lane_v carries the offset of the V region
    auto v_frag = [&](int f) {  // fragment f: 32-key chunk f/8, d tile f%8; keys 4q .. 4q + 3 of both 16-key halves
      const uint8_t* src = sV + lane_v[f & 7] + (f >> 3) * 32 * 256;
      const v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4i16*)src);
      const v4i16 hi =
          __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4i16*)(src + 16 * 256));
      const v8i16 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      return __builtin_bit_cast(bf16x8, both);
    };
    // operand fragments are read kAhead fragments before their use; the last slots of stage 1 already fetch
    // the first V^T fragments of stage 2 (block kb landed long ago), so only stage 1 starts cold
    bf16x8 kf[kAhead + 1], vf[kAhead + 1];
#pragma unroll
    for (int f = 0; f < kAhead; ++f) kf[f] = k_frag(f);
    int n = kExpEarly;
#pragma unroll
    for (int f = 0; f < 16; ++f) {
      if (f + kAhead < 16)
        kf[(f + kAhead) % (kAhead + 1)] = k_frag(f + kAhead);
      else
        vf[(f + kAhead - 16) % (kAhead + 1)] = v_frag(f + kAhead - 16);
      const int dc = f >> 2, kt = f & 3;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        s_next[kt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[f % (kAhead + 1)], qf[t][dc],
                                                                dc == 0 ? zero4 : s_next[kt][t], 0, 0, 0);
        // 32 - kExpEarly entries over 32 slots: one per slot until they are done
        if (n < 32) exp_entry(s_cur, pw_cur, n++);
        if (t == 0 && f == kLoadSlots[0]) issue_piece((stage + 3) % kStages, 0);
        if (t == 0 && f == kLoadSlots[1]) issue_piece((stage + 3) % kStages, 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      l_run[t] += lsum[t][0] + lsum[t][1];
      lsum[t][0] = lsum[t][1] = 0.f;
    }
    // ---- stage 2: O^T += V^T P^T, 16 operand fragments = [transposing LDS reads of a V^T operand, two MFMAs]
    auto pv_frag = [&](int f, int t) {
      if (t == 0 && f + kAhead < 16) vf[(f + kAhead) % (kAhead + 1)] = v_frag(f + kAhead);
      const int ch = f >> 3, dt = f & 7;
      const u32x4 w = {pw_cur[ch][t][0], pw_cur[ch][t][1], pw_cur[ch][t][2], pw_cur[ch][t][3]};
      oacc[dt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[f % (kAhead + 1)], __builtin_bit_cast(bf16x8, w),
                                                            oacc[dt][t], 0, 0, 0);
    };
    constexpr int kScanFrags = 4;  // PV fragments issued before the block maximum of S(kb+1) is looked at
#pragma unroll
    for (int f = 0; f < kScanFrags; ++f)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        pv_frag(f, t);
        __builtin_amdgcn_sched_barrier(0);
      }
    if (__builtin_expect(kb + 1 < kb_end, 1)) {
      mask_tail(s_next, kb + 1);
      float mx[2] = {0.f, 0.f};
      if (SCAN) ref_scan(s_next, mx);
      if (SCAN && __builtin_expect(ref_must_move(mx, kb + 1), 0)) {
        // rare: O, l and the scores of block kb+1 move to the new reference now; the part of P(kb) that
        // the remaining PV MFMAs still have to accumulate follows (one more bf16 rounding on it)
        float alpha[2];
        ref_move(s_next, mx, kb + 1, alpha);
#pragma unroll
        for (int ch = 0; ch < 2; ++ch)
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              uint32_t& word = pw_cur[ch][t][w];
              word = pack_bf16x2(bf16_lo(word) * alpha[t], bf16_hi(word) * alpha[t]);
            }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // (in the last interval the entries below come from a block that does not exist and are dropped)
    int n2 = 0;
#pragma unroll
    for (int f = kScanFrags; f < 16; ++f)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        pv_frag(f, t);
        // kExpEarly entries over the 2 (16 - kScanFrags) remaining slots: every second slot
        if (t == 0 && n2 < kExpEarly) exp_entry(s_next, pw_next, n2++);
        if (t == 1 && f == kLoadSlots[2]) issue_piece((stage + 3) % kStages, 2);
        if (t == 1 && f == kLoadSlots[3]) issue_piece((stage + 3) % kStages, 3);
        __builtin_amdgcn_sched_barrier(0);
      }
  };

  f32x4 sA[4][2], sB[4][2];
  uint32_t pwA[2][2][4], pwB[2][2][4];
  __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8): block 0 has landed
  __builtin_amdgcn_s_barrier();
  qk(sA, 0);
  {
    mask_tail(sA, kb_begin);
    if (SCAN) {
      float mx[2], alpha[2];
      ref_scan(sA, mx);
      if (ref_must_move(mx, kb_begin)) ref_move(sA, mx, kb_begin, alpha);
    }
#pragma unroll
    for (int n = 0; n < kExpEarly; ++n) exp_entry(sA, pwA, n);
  }
  for (int kb = kb_begin; kb < kb_end; kb += 4) {  // stage of block kb = (kb - kb_begin) % 4
    interval(kb, 0, sA, sB, pwA, pwB);
    if (kb + 1 < kb_end) interval(kb + 1, 1, sB, sA, pwB, pwA);
    if (kb + 2 < kb_end) interval(kb + 2, 2, sA, sB, pwA, pwB);
    if (kb + 3 < kb_end) interval(kb + 3, 3, sB, sA, pwB, pwA);
  }
  __builtin_amdgcn_s_waitcnt(0);  // drain trailing async loads

  // ---- lane (q, i): queries 16t + i, d = 16dt + 4q + e
  float l_row[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) l_row[t] = quad_sum(l_run[t]);
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int64_t row = q0 + t * 16 + i16;
    if (row < Sq) store_output(p, b, h, row, q4, oacc, t, 1.0f / l_row[t]);
  }
}

}  // namespace

// One workgroup per (batch, head, 256-query block); no scratch, no key split.  `units` as launch_attn_plain counts them.
int launch_attn_plain16(const dsx_attn_params& p, int64_t units, hipStream_t st) {
  static PerDeviceOnce attr_once;
  const int attr_rc = per_device_once(attr_once, [](int) {
    if (hipFuncSetAttribute((const void*)attn_plain16_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_plain16_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
      return (int)DSX_ELAUNCH;
    return (int)DSX_OK;
  });
  if (attr_rc != DSX_OK) return attr_rc;
  if (units > (1ll << 30)) return DSX_EBADSHAPE;
  const dim3 grid((unsigned)(((units + 7) / 8) * 8)), block(512);
  const bool bounded = p.score_bound > 0.f && p.score_bound * kLog2e <= kRescaleThreshold;
  if (p.qk_norm2_max && !bounded) {
    // the bound lives on the device: launch both variants, each looks at it and one of them returns at once
    attn_plain16_kernel<false><<<grid, block, kLdsBytes, st>>>(p, (int)units, 1);
    attn_plain16_kernel<true><<<grid, block, kLdsBytes, st>>>(p, (int)units, 1);
  } else if (bounded) {
    attn_plain16_kernel<false><<<grid, block, kLdsBytes, st>>>(p, (int)units, 0);
  } else {
    attn_plain16_kernel<true><<<grid, block, kLdsBytes, st>>>(p, (int)units, 0);
  }
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}

}  // namespace dsx
