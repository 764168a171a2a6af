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
// The product is skinny (rank <= 128) and HBM-bound on reading xq once: one workgroup owns 32 token rows, its
// wavefronts split K between them (v_mfma_f32_32x32x64_f8f6f4 on operands loaded straight from global memory) and
// add their partial sums through LDS in a fixed order, so the result does not depend on timing.
#include "common.h"

namespace dsx {

template <int NT>  // rank tiles of 32
__global__ __launch_bounds__(1024) void lora_down_kernel(const uint8_t* __restrict__ a, int64_t lda,
                                                         const uint8_t* __restrict__ d, int64_t ldd,
                                                         const float* __restrict__ row_scale, uint8_t* __restrict__ out,
                                                         int64_t ldo, int M, int K, int ranks, int copies, int E) {
  extern __shared__ __attribute__((aligned(16))) float red[];  // [wave][tile][16][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int g = lane >> 5, li = lane & 31;
  const int m0 = blockIdx.x * 32;
  const int steps = K >> 6;
  const int s0 = (int)((int64_t)steps * wave / nw), s1 = (int)((int64_t)steps * (wave + 1) / nw);
  const uint8_t* ap = a + (int64_t)min(m0 + li, M - 1) * lda + g * 32;
  const uint8_t* dp = d + (int64_t)li * ldd + g * 32;
  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
#pragma unroll 3
  for (int s = s0; s < s1; ++s) {
    const i32x4 a0 = *reinterpret_cast<const i32x4*>(ap + (int64_t)s * 64);
    const i32x4 a1 = *reinterpret_cast<const i32x4*>(ap + (int64_t)s * 64 + 16);
    const i32x8 af = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const uint8_t* dt = dp + (int64_t)t * 32 * ldd + (int64_t)s * 64;
      const i32x4 d0 = *reinterpret_cast<const i32x4*>(dt);
      const i32x4 d1 = *reinterpret_cast<const i32x4*>(dt + 16);
      const i32x8 df = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
      acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(df, af, acc[t], 0, 0, 0, 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) red[((wave * NT + t) * 16 + r) * 64 + lane] = acc[t][r];
  __syncthreads();
  // lane (g, li) of tile t: token m0 + li, ranks 32t + 8rq + 4g + e
  for (int item = threadIdx.x; item < NT * 64; item += blockDim.x) {
    const int t = item >> 6, l = item & 63, lg = l >> 5, lli = l & 31;
    const int m = m0 + lli;
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float s = 0.f;
        for (int w = 0; w < nw; ++w) s += red[((w * NT + t) * 16 + 4 * rq + e) * 64 + l];
        const int rank = t * 32 + 8 * rq + 4 * lg + e;
        v[e] = fminf(fmaxf(s * row_scale[rank], -448.f), 448.f);
      }
      const int rank0 = t * 32 + 8 * rq + 4 * lg;
      if (m < M && rank0 < ranks) {  // (rows of d from `ranks` on are padding)
        const uint32_t codes = pack_e4m3x4_inrange(v[0], v[1], v[2], v[3]);
        for (int c = 0; c < copies; ++c)
          *reinterpret_cast<uint32_t*>(out + (int64_t)m * ldo + c * ranks + rank0) = codes;
      }
    }
  }
  // columns from the last copy up to E: zero codes (the extension weight's columns there are zero as well, and
  // 0 x NaN would still be NaN)
  const int filled = copies * ranks;
  const int zero_words = (E - filled) >> 2;
  for (int item = threadIdx.x; item < 32 * zero_words; item += blockDim.x) {
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
  if (M < 0 || M > (1 << 30) || K <= 0 || K > (1 << 30) || (K & 63) || R <= 0 || R > 128 || (R & 31) || ranks <= 0 ||
      ranks > R || (ranks & 3) || copies < 1 || copies > 32 || E < ranks * copies || E > (1 << 20) || (E & 15) ||
      lda < K || ldd < K || ldo < E)
    return DSX_EBADSHAPE;
  if ((lda & 15) || (ldd & 15) || (ldo & 15) || ((uintptr_t)a & 15) || ((uintptr_t)d & 15) || ((uintptr_t)out & 15) ||
      ((uintptr_t)row_scale & 3))
    return DSX_EALIGN;
  const int nt = (int)(R / 32);
  // wavefronts per workgroup: about six 64-byte steps of K each (the loads of a wave's steps are in flight
  // together), at most sixteen and at most what 128 KiB of partial sums hold
  const int steps = (int)(K >> 6);
  int nw = (steps + 5) / 6;
  nw = nw < 1 ? 1 : (nw > 16 ? 16 : nw);
  while (nw * nt > 32) --nw;
  const size_t lds = (size_t)nw * nt * 16 * 64 * sizeof(float);
  static PerDeviceOnce once;
  const int rc = per_device_once(once, [](int) {
    const void* kernels[4] = {(const void*)lora_down_kernel<1>, (const void*)lora_down_kernel<2>,
                              (const void*)lora_down_kernel<3>, (const void*)lora_down_kernel<4>};
    for (const void* k : kernels)
      if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) != hipSuccess)
        return (int)DSX_ELAUNCH;
    return (int)DSX_OK;
  });
  if (rc != DSX_OK) return rc;
  const dim3 grid((unsigned)((M + 31) / 32)), block((unsigned)(64 * nw));
  hipStream_t st = (hipStream_t)stream;
#define DSX_LAUNCH(NT)                                                                                              \
  lora_down_kernel<NT><<<grid, block, lds, st>>>((const uint8_t*)a, lda, (const uint8_t*)d, ldd, row_scale,          \
                                                 (uint8_t*)out, ldo, (int)M, (int)K, (int)ranks, (int)copies, (int)E)
  switch (nt) {
    case 1: DSX_LAUNCH(1); break;
    case 2: DSX_LAUNCH(2); break;
    case 3: DSX_LAUNCH(3); break;
    default: DSX_LAUNCH(4); break;
  }
#undef DSX_LAUNCH
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}
