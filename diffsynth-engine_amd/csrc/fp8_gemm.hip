// FP8 e4m3 scaled GEMM for gfx950:  out = bf16((A * W^T) * a_scale[m] * w_scale + bias[n]).
//
// Both operands are K-contiguous ("TN"), which is what v_mfma_f32_32x32x64_f8f6f4 wants: lane
// (g = lane/32, i = lane%32) feeds 32 consecutive K bytes of row i for the A operand and of
// column i for the B operand.  Any permutation of K that is applied to both operands leaves
// the product unchanged, so the tile loader only has to keep the two consistent.
//
// Tiling: 256x256 output tile per workgroup, 4 waves as 2x2, each wave 128x128 = 4x4 MFMA
// tiles (256 fp32 accumulator registers), K step 128 bytes, two LDS stages (2 x 64 KiB).
// LDS rows are 128 B (8 chunks of 16 B); chunk c of row r is stored at chunk c ^ ((r/2)&7) so
// that 16 lanes reading 16 consecutive rows at the same logical chunk hit 16 distinct
// 16-byte bank groups.
#include "common.h"

namespace dsx {

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kStageBytes = (BM + BN) * BK;  // 64 KiB

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
};

__device__ __forceinline__ void tile_coords(int wg, int tiles_m, int tiles_n, int& tm, int& tn,
                                            bool& valid) {
  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of
  // logical tile ids so that tiles sharing A rows / W rows meet in the same L2.
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + 7) >> 3;
  const int L = (wg & 7) * per_xcd + (wg >> 3);
  valid = L < total;
  const int G = 4;
  const int span = G * tiles_n;
  const int group = L / span;
  const int first_m = group * G;
  const int gsz = min(tiles_m - first_m, G);
  const int rem = L - group * span;
  tm = first_m + rem % gsz;
  tn = rem / gsz;
}

__global__ __launch_bounds__(256) void fp8_gemm_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int tm, tn;
  bool valid;
  tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn, valid);
  if (!valid) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int g = lane >> 5, li = lane & 31;
  const int m0 = tm * BM, n0 = tn * BN;
  const int kchunks = p.K >> 4;  // 16-byte chunks per row

  // --- global -> register staging: thread handles chunks id = tid + 256*i, i < 8, per operand
  const int st_c = tid & 7;        // chunk within the 128-byte K slab
  const int st_r = tid >> 3;       // row 0..31 (+32*i)
  const uint8_t* a_src[8];
  const uint8_t* w_src[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int ra = min(m0 + st_r + 32 * i, p.M - 1);
    int rw = min(n0 + st_r + 32 * i, p.N - 1);
    a_src[i] = p.a + (int64_t)ra * p.lda + st_c * 16;
    w_src[i] = p.w + (int64_t)rw * p.ldw + st_c * 16;
  }
  int st_off[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) st_off[i] = lds_off(st_r + 32 * i, st_c);

  u32x4 sa[8], sw[8];
  auto load_stage = [&](int kt) {
    const bool in = (kt * 8 + st_c) < kchunks;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      sa[i] = in ? *reinterpret_cast<const u32x4*>(a_src[i] + (int64_t)kt * BK) : u32x4{0, 0, 0, 0};
      sw[i] = in ? *reinterpret_cast<const u32x4*>(w_src[i] + (int64_t)kt * BK) : u32x4{0, 0, 0, 0};
    }
  };
  auto store_stage = [&](int buf) {
    uint8_t* sA = smem + buf * kStageBytes;
    uint8_t* sB = sA + BM * BK;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      *reinterpret_cast<u32x4*>(sA + st_off[i]) = sa[i];
      *reinterpret_cast<u32x4*>(sB + st_off[i]) = sw[i];
    }
  };

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = (p.K + BK - 1) / BK;
  load_stage(0);
  store_stage(0);
  __syncthreads();

  // per-lane LDS row bases of the fragments this wave reads
  const int a_row = wm * 128 + li;
  const int b_row = wn * 128 + li;

  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_stage(kt + 1);
    const uint8_t* sA = smem + buf * kStageBytes;
    const uint8_t* sB = sA + BM * BK;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      i32x8 fa[4], fb[4];
      const int c0 = ks * 4 + g * 2;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int ra = a_row + t * 32, rb = b_row + t * 32;
        i32x4 a_lo = *reinterpret_cast<const i32x4*>(sA + lds_off(ra, c0));
        i32x4 a_hi = *reinterpret_cast<const i32x4*>(sA + lds_off(ra, c0 + 1));
        i32x4 b_lo = *reinterpret_cast<const i32x4*>(sB + lds_off(rb, c0));
        i32x4 b_hi = *reinterpret_cast<const i32x4*>(sB + lds_off(rb, c0 + 1));
        fa[t] = i32x8{a_lo.x, a_lo.y, a_lo.z, a_lo.w, a_hi.x, a_hi.y, a_hi.z, a_hi.w};
        fb[t] = i32x8{b_lo.x, b_lo.y, b_lo.z, b_lo.w, b_hi.x, b_hi.y, b_hi.z, b_hi.w};
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], 0, 0,
                                                                      0, 0, 0, 0);
    }
    if (kt + 1 < nk) store_stage(buf ^ 1);
    __syncthreads();
  }

  // --- epilogue.  C layout of a 32x32 tile: lane (g, li) register r holds
  //     row 8*(r/4) + 4*g + (r%4), column li.
  const float ws = p.w_scale ? *p.w_scale : 1.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = n0 + wn * 128 + j * 32 + li;
    const bool col_ok = col < p.N;
    const float bj = (p.bias && col_ok) ? bf16_bits_to_f32(p.bias[col]) : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (col_ok && row < p.M) {
          const float as = p.a_scale ? p.a_scale[row] : 1.0f;
          float v = acc[i][j][r] * (as * ws) + bj;
          p.out[(int64_t)row * p.ldo + col] = (uint16_t)f32_to_bf16_bits(v);
        }
      }
    }
  }
}

// Small-M path (M <= 8): one wave per output column, fp32 FMA over dequantised bytes.
// HBM-bound on the weight read; used for the M=1 conditioning projections.
__global__ __launch_bounds__(256) void fp8_gemv_kernel(GemmArgs p) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= p.N) return;
  const int kchunks = p.K >> 4;
  float acc[8];
#pragma unroll
  for (int m = 0; m < 8; ++m) acc[m] = 0.f;
  const u32x4* wr = reinterpret_cast<const u32x4*>(p.w + (int64_t)n * p.ldw);
  for (int c = lane; c < kchunks; c += 64) {
    u32x4 wv = __builtin_nontemporal_load(wr + c);
    float wf[16];
#pragma unroll
    for (int b = 0; b < 16; ++b) wf[b] = e4m3_bits_to_f32((wv[b >> 2] >> ((b & 3) * 8)) & 0xffu);
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      if (m < p.M) {
        u32x4 av = *reinterpret_cast<const u32x4*>(p.a + (int64_t)m * p.lda + c * 16);
#pragma unroll
        for (int b = 0; b < 16; ++b)
          acc[m] += wf[b] * e4m3_bits_to_f32((av[b >> 2] >> ((b & 3) * 8)) & 0xffu);
      }
    }
  }
  const float ws = p.w_scale ? *p.w_scale : 1.0f;
  const float bj = p.bias ? bf16_bits_to_f32(p.bias[n]) : 0.f;
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    if (m < p.M) {
      float s = wave_sum(acc[m]);
      if (lane == 0) {
        const float as = p.a_scale ? p.a_scale[m] : 1.0f;
        p.out[(int64_t)m * p.ldo + n] = (uint16_t)f32_to_bf16_bits(s * (as * ws) + bj);
      }
    }
  }
}

}  // namespace dsx

extern "C" int dsx_fp8_gemm(const void* a, int64_t lda, const void* w, int64_t ldw,
                            const float* a_scale, const float* w_scale, const void* bias, void* out,
                            int64_t ldo, int64_t M, int64_t N, int64_t K, void* stream) {
  using namespace dsx;
  if (!a || !w || !out) return DSX_ENULL;
  if (M < 0 || N <= 0 || K <= 0 || (K & 15) || lda < K || ldw < K || ldo < N) return DSX_EBADSHAPE;
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return DSX_EBADSHAPE;
  if ((lda & 15) || (ldw & 15) || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || ((uintptr_t)out & 1))
    return DSX_EALIGN;
  if (M == 0) return DSX_OK;
  GemmArgs p;
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
  hipStream_t st = (hipStream_t)stream;
  if (M <= 8) {
    p.tiles_m = p.tiles_n = 0;
    fp8_gemv_kernel<<<dim3((unsigned)((N + 3) / 4)), dim3(256), 0, st>>>(p);
    return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
  }
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  const int total = p.tiles_m * p.tiles_n;
  const int grid = ((total + 7) / 8) * 8;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)fp8_gemm_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            2 * kStageBytes) != hipSuccess)
      return DSX_ELAUNCH;
    attr_set = true;
  }
  fp8_gemm_kernel<<<dim3((unsigned)grid), dim3(256), 2 * kStageBytes, st>>>(p);
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}
