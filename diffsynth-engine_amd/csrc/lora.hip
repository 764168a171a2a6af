// Down projection of unfused low-rank updates (LoRALinear.forward, diffsynth_engine/models/basic/lora.py:29-32,137-141),
// emitted as the extension operand of the main product:
//
//   y = x W^T + c up(down(x))  =  s_x[m] s_w ( sum_k xq[m,k] wq[n,k]  +  sum_r t[m,r] u[n,r] ),
//   t[m,r] = e4m3( row_scale[r] * sum_k xq[m,k] dq[r,k] ),   u = e4m3( c U / (s_w s_u) ),   row_scale = s_d s_u,
//
// so the low-rank term rides the main GEMM as 128 more columns of its reduction axis (dsx_gemm_problem.a_ext /
// w_ext) instead of a second product and a pass over the output.  The activation's per-token scale is NOT applied
// here: the main product applies it to the whole extended sum.  Values beyond e4m3's 448 saturate; to keep them
// away from it the values of a row can be written `copies` times side by side (the caller repeats the columns of
// u and folds 1 / copies into row_scale): the few terms of a low-rank product would otherwise have to be as large,
// each, as the sum of K terms they sit beside.
//
// The product is skinny (rank <= 128) and bound by reading xq once.  One workgroup owns 16 token rows; its
// wavefronts deal the 128-byte chunks of K between them, and every wavefront runs a pipeline of its own: its chunk
// of the activation rows and of the stacked down factors goes HBM/L2 -> LDS with global_load_lds_dwordx4 (eight
// whole 128-byte lines per instruction; loading MFMA fragments straight from global memory touches 32 lines for
// 1 KiB, overfills the vector L1 fourfold and was 2-3 times slower), up to three chunks in flight per wavefront
// and no workgroup barrier in the loop, then v_mfma_f32_16x16x128_f8f6f4 on fragments read back with the row
// swizzle of the main GEMM.  The wavefronts' partial sums meet in LDS in a fixed order, so the result does not
// depend on timing.
#include "common.h"

namespace dsx {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt immediate for vmcnt(vm), lgkmcnt and expcnt left alone
constexpr int lora_vmcnt_imm(int vm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (15 << 8); }

template <int NR16, int NB>  // rank tiles of 16; chunk buffers per wavefront
__global__ __launch_bounds__(512) void lora_down_kernel(const uint8_t* __restrict__ a, int64_t lda,
                                                        const uint8_t* __restrict__ d, int64_t ldd,
                                                        const float* __restrict__ row_scale, uint8_t* __restrict__ out,
                                                        int64_t ldo, int M, int K, int ranks, int copies, int E) {
  constexpr int kTile = 16 * 128;                // one 16-row tile of a 128-byte chunk
  constexpr int kBuf = kTile * (1 + NR16);       // activation tile, then the rank tiles
  constexpr int kLoads = 2 * (1 + NR16);         // async load instructions per chunk (8 rows each)
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int m0 = blockIdx.x * 16;
  const int chunks = K >> 7;
  const int mine = (chunks - wave + nw - 1) / nw;  // chunks wave, wave + nw, ... (>= 0)

  // async loads: lane l of an instruction fills LDS bytes [16 l, 16 l + 16) of its 1 KiB destination, i.e. 16-byte
  // position l % 8 of row l / 8; position p of row r holds the row's chunk p ^ ((r / 2) & 7) (the main GEMM's swizzle)
  const int ld_r = lane >> 3, ld_p = lane & 7;
  uint32_t a_off[2], d_off[2 * NR16];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = 8 * i + ld_r;
    a_off[i] = (uint32_t)(min(m0 + row, M - 1) - m0) * (uint32_t)lda + ((ld_p ^ ((row >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int i = 0; i < 2 * NR16; ++i) {
    const int row = 8 * i + ld_r;
    d_off[i] = (uint32_t)row * (uint32_t)ldd + ((ld_p ^ ((row >> 1) & 7)) << 4);
  }
  const uint8_t* a_base = a + (int64_t)m0 * lda;
  const uint32_t lds_wave = (uint32_t)(uintptr_t)(lds_ptr_t)smem + (uint32_t)wave * (NB * kBuf);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  auto issue = [&](int k) {  // this wavefront's k-th chunk into buffer k % NB
    const int64_t byte0 = (int64_t)(wave + k * nw) << 7;
    const uint32_t dst = lds_wave + (uint32_t)(k % NB) * kBuf;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(a_off[i]), "s"(a_base + byte0), "s"(dst + i * 1024)
                   : "memory", "m0");
#pragma unroll
    for (int i = 0; i < 2 * NR16; ++i)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(d_off[i]), "s"(d + byte0), "s"(dst + kTile + i * 1024)
                   : "memory", "m0");
  };
#pragma clang diagnostic pop

  // fragments of v_mfma_f32_16x16x128_f8f6f4: lane (q = lane / 16, i = lane % 16) holds bytes [32 q, 32 q + 32) of
  // row i of a tile, i.e. its chunks 2 q and 2 q + 1
  const int q16 = lane >> 4, i16 = lane & 15;
  uint32_t frag[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) frag[h] = (uint32_t)(i16 * 128 + (((2 * q16 + h) ^ ((i16 >> 1) & 7)) << 4));
  f32x4 acc[NR16];
#pragma unroll
  for (int r = 0; r < NR16; ++r)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[r][e] = 0.f;

#pragma unroll
  for (int k = 0; k < NB - 1; ++k)
    if (k < mine) issue(k);
  for (int k = 0; k < mine; ++k) {
    if (k + NB - 1 < mine) issue(k + NB - 1);  // into the buffer chunk k - 1 was read from (its MFMAs are issued)
    const int ahead = min(NB - 1, mine - 1 - k);  // chunks issued after chunk k
    if (ahead >= 2)
      __builtin_amdgcn_s_waitcnt(lora_vmcnt_imm(2 * kLoads));
    else if (ahead == 1)
      __builtin_amdgcn_s_waitcnt(lora_vmcnt_imm(kLoads));
    else
      __builtin_amdgcn_s_waitcnt(lora_vmcnt_imm(0));
    asm volatile("" ::: "memory");  // the reads below stay behind the wait
    const uint8_t* buf = smem + (size_t)wave * (NB * kBuf) + (size_t)(k % NB) * kBuf;
    const i32x4 a0 = *reinterpret_cast<const i32x4*>(buf + frag[0]);
    const i32x4 a1 = *reinterpret_cast<const i32x4*>(buf + frag[1]);
    const i32x8 af = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
    for (int r = 0; r < NR16; ++r) {
      const i32x4 d0 = *reinterpret_cast<const i32x4*>(buf + kTile + r * kTile + frag[0]);
      const i32x4 d1 = *reinterpret_cast<const i32x4*>(buf + kTile + r * kTile + frag[1]);
      const i32x8 df = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
      // first operand: ranks, second: tokens -> lane (q, i) holds token i and ranks 16 r + 4 q .. + 3
      acc[r] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(df, af, acc[r], 0, 0, 0, 0, 0, 0);
    }
    asm volatile("" ::: "memory");  // the next round's load into this buffer stays behind these reads
  }

  // partial sums of the wavefronts, added in wavefront order
  float* red = reinterpret_cast<float*>(smem);  // [wave][rank tile][4][64]
  __syncthreads();                              // every wavefront is done with its chunk buffers
#pragma unroll
  for (int r = 0; r < NR16; ++r)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[((wave * NR16 + r) * 4 + e) * 64 + lane] = acc[r][e];
  __syncthreads();
  for (int item = threadIdx.x; item < NR16 * 64; item += blockDim.x) {
    const int r = item >> 6, l = item & 63, lq = l >> 4, li = l & 15;
    const int m = m0 + li, rank0 = 16 * r + 4 * lq;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float s = 0.f;
      for (int w = 0; w < nw; ++w) s += red[((w * NR16 + r) * 4 + e) * 64 + l];
      v[e] = fminf(fmaxf(s * row_scale[rank0 + e], -448.f), 448.f);
    }
    if (m < M && rank0 < ranks) {  // (rows of d from `ranks` on are padding)
      const uint32_t codes = pack_e4m3x4_inrange(v[0], v[1], v[2], v[3]);
      for (int c = 0; c < copies; ++c)
        *reinterpret_cast<uint32_t*>(out + (int64_t)m * ldo + c * ranks + rank0) = codes;
    }
  }
  // columns from the last copy up to E: zero codes (the extension weight's columns there are zero as well, and
  // 0 x NaN would still be NaN)
  const int filled = copies * ranks;
  const int zero_words = (E - filled) >> 2;
  for (int item = threadIdx.x; item < 16 * zero_words; item += blockDim.x) {
    const int r = item / zero_words, c = item - r * zero_words;
    if (m0 + r < M) *reinterpret_cast<uint32_t*>(out + (int64_t)(m0 + r) * ldo + filled + c * 4) = 0u;
  }
}

}  // namespace dsx

extern "C" int dsx_lora_down(const void* a, int64_t lda, const void* d, int64_t ldd, const float* row_scale,
                             void* out, int64_t ldo, int64_t M, int64_t K, int64_t R, int64_t ranks, int64_t copies,
                             int64_t E, void* stream) {
  using namespace dsx;
  if (M == 0) return (K <= 0 || R <= 0) ? DSX_EBADSHAPE : DSX_OK;
  if (!a || !d || !row_scale || !out) return DSX_ENULL;
  if (M < 0 || M > (1 << 30) || K <= 0 || K > (1 << 30) || (K & 127) || R <= 0 || R > 128 || (R & 31) || ranks <= 0 ||
      ranks > R || (ranks & 3) || copies < 1 || copies > 32 || E < ranks * copies || E > (1 << 20) || (E & 15) ||
      lda < K || ldd < K || ldo < E || lda >= (1 << 24) || ldd >= (1 << 24))  // (per-lane load offsets are 32-bit)
    return DSX_EBADSHAPE;
  if ((lda & 15) || (ldd & 15) || (ldo & 15) || ((uintptr_t)a & 15) || ((uintptr_t)d & 15) || ((uintptr_t)out & 15) ||
      ((uintptr_t)row_scale & 3))
    return DSX_EALIGN;
  const int nr16 = (int)((ranks + 15) / 16);  // rank tiles that hold a real rank (rows of d up to 16 nr16 <= R exist)
  const int nb = nr16 <= 2 ? 3 : 2;
  const int buf_bytes = 2048 * (1 + nr16);
  // wavefronts: at most eight, at most one per chunk, at most what 128 KiB of chunk buffers hold
  const int chunks = (int)(K >> 7);
  int nw = chunks < 8 ? chunks : 8;
  while (nw > 1 && nw * nb * buf_bytes > 128 * 1024) --nw;
  size_t lds = (size_t)nw * nb * buf_bytes;
  const size_t red_bytes = (size_t)nw * nr16 * 4 * 64 * sizeof(float);
  if (red_bytes > lds) lds = red_bytes;
  const dim3 grid((unsigned)((M + 15) / 16)), block((unsigned)(64 * nw));
  hipStream_t st = (hipStream_t)stream;
  static PerDeviceOnce once;
#define DSX_LORA_FORMS(X) X(1, 3) X(2, 3) X(3, 2) X(4, 2) X(5, 2) X(6, 2) X(7, 2) X(8, 2)
  const int rc = per_device_once(once, [](int) {
#define DSX_ATTR(NR, NB)                                                                                          \
  if (hipFuncSetAttribute((const void*)lora_down_kernel<NR, NB>, hipFuncAttributeMaxDynamicSharedMemorySize,     \
                          128 * 1024) != hipSuccess)                                                              \
    return (int)DSX_ELAUNCH;
    DSX_LORA_FORMS(DSX_ATTR)
#undef DSX_ATTR
    return (int)DSX_OK;
  });
  if (rc != DSX_OK) return rc;
  switch (nr16) {
#define DSX_CASE(NR, NB)                                                                                          \
  case NR:                                                                                                        \
    lora_down_kernel<NR, NB><<<grid, block, lds, st>>>((const uint8_t*)a, lda, (const uint8_t*)d, ldd, row_scale, \
                                                       (uint8_t*)out, ldo, (int)M, (int)K, (int)ranks,            \
                                                       (int)copies, (int)E);                                      \
    break;
    DSX_LORA_FORMS(DSX_CASE)
#undef DSX_CASE
    default: return DSX_EBADSHAPE;
  }
#undef DSX_LORA_FORMS
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}
