// Library-level entry points: ABI version, error strings, device check.
#include <string.h>

#include <type_traits>

#include "common.h"

extern "C" int dsx_abi_version(void) { return DSX_ABI_VERSION; }

extern "C" const char* dsx_strerror(int code) {
  switch (code) {
    case DSX_OK: return "ok";
    case DSX_EBADSHAPE: return "unsupported shape, size or stride";
    case DSX_EALIGN: return "pointer, stride or leading dimension is not suitably aligned";
    case DSX_EARCH: return "current device is not gfx950 (MI355X)";
    case DSX_ELAUNCH: return "kernel launch failed";
    case DSX_ENULL: return "required pointer is NULL";
    case DSX_EWORKSPACE: return "scratch memory missing or too small for this call";
    default: return "unknown dsx error code";
  }
}

extern "C" int dsx_check_device(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return DSX_EARCH;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return DSX_EARCH;
  return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? DSX_OK : DSX_EARCH;
}

// ---- on-box microbenchmark of the matrix pipe: MFMAs on register operands in a loop, no memory traffic --------
// What the chip sustains with nothing but matrix instructions in flight, for the operand bits the caller supplies
// (all-zero operands run at the full clock; random bits draw more power and the clock management lowers the clock).
namespace dsx {
// KIND 0 / 1: v_mfma_f32_32x32x16_bf16 / v_mfma_scale_f32_32x32x64_f8f6f4 (sixteen accumulator registers each);
// KIND 2 / 3: v_mfma_f32_16x16x32_bf16 / v_mfma_scale_f32_16x16x128_f8f6f4 (four accumulator registers each, eight
// independent accumulators, so that a wavefront has the same number of MFMAs in flight between two uses of one).
template <int KIND, bool ROT = false>
__global__ __launch_bounds__(256) void mfma_ceiling_kernel(const uint32_t* __restrict__ bits, int64_t iters,
                                                           float* __restrict__ sink) {
  // eight operand dwords per lane and operand (bf16: 4 + 4 are used; fp8: 8 + 8), the same for every workgroup
  uint32_t r[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) r[i] = bits[i * 256 + threadIdx.x];
  constexpr bool kSmall = KIND >= 2;
  constexpr int kAcc = kSmall ? 8 : 4;
  typedef typename std::conditional<kSmall, f32x4, f32x16>::type acc_t;
  acc_t acc[kAcc];
#pragma unroll
  for (int t = 0; t < kAcc; ++t)
#pragma unroll
    for (int e = 0; e < (kSmall ? 4 : 16); ++e) acc[t][e] = 0.f;
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int t = 0; t < kAcc; ++t) {  // independent accumulators
      const int ra = ROT ? (t & 3) : 0;  // ROT: the first operand changes from one MFMA to the next as well
      const int tb = t & 3;
      if constexpr (KIND == 0 || KIND == 2) {
        const u32x4 a = {r[ra], r[ra + 1], r[ra + 2], r[ra + 3]}, b = {r[8 + tb], r[9 + tb], r[10 + tb], r[11 + tb]};
        if constexpr (KIND == 0)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                           acc[t], 0, 0, 0);
        else  // as assembly with the accumulator tied to itself: for this shape the compiler's own allocation puts
              // source and destination accumulators in different registers and copies them around once per round
          asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[t]) : "v"(a), "v"(b));
      } else {
        const i32x8 a = {(int)r[ra], (int)r[ra + 1], (int)r[ra + 2], (int)r[ra + 3], (int)r[ra + 4], (int)r[ra + 5],
                         (int)r[ra + 6], (int)r[ra + 7]};
        const i32x8 b = {(int)r[8], (int)r[9], (int)r[10], (int)r[11], (int)r[12 + (tb & 1)], (int)r[13], (int)r[14],
                         (int)r[15 - (tb >> 1)]};
        if constexpr (KIND == 1)
          acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[t], 0, 0, 0, 0, 0, 0);
        else
          acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[t], 0, 0, 0, 0, 0, 0);
      }
    }
  }
  if constexpr (KIND == 2) asm volatile("s_nop 15\n\ts_nop 15");  // (the assembly MFMAs' results, before they are read)
  float s = 0.f;
#pragma unroll
  for (int t = 0; t < kAcc; ++t)
#pragma unroll
    for (int e = 0; e < (kSmall ? 4 : 16); ++e) s += acc[t][e];
  if (s == 12345.678f) sink[0] = s;  // keeps the loop alive; never true for the inputs of the probe
}
}  // namespace dsx

extern "C" int dsx_mfma_ceiling_probe(int kind, const void* operand_bits, int64_t iters, int32_t workgroups,
                                      void* sink, int64_t* flops_out, void* stream) {
  if (!operand_bits || !sink) return DSX_ENULL;
  // Caps: 2^22 iterations of four dependent MFMAs on 2^14 workgroups are already seconds of work; anything larger
  // would keep the device busy for minutes, which callers sharing it cannot tell from a hang.
  if (kind < 0 || kind > 7 || iters <= 0 || iters > DSX_PROBE_MAX_ITERS || workgroups <= 0 ||
      workgroups > DSX_PROBE_MAX_WORKGROUPS)
    return DSX_EBADSHAPE;
  if ((uintptr_t)operand_bits & 3) return DSX_EALIGN;
  const dim3 grid((unsigned)workgroups), block(256);
  hipStream_t st = (hipStream_t)stream;
#define DSX_PROBE(K, R) dsx::mfma_ceiling_kernel<K, R><<<grid, block, 0, st>>>((const uint32_t*)operand_bits, iters, (float*)sink)
  switch (kind) {
    case 0: DSX_PROBE(0, false); break;
    case 1: DSX_PROBE(1, false); break;
    case 2: DSX_PROBE(2, false); break;
    case 3: DSX_PROBE(3, false); break;
    case 4: DSX_PROBE(0, true); break;
    case 5: DSX_PROBE(1, true); break;
    case 6: DSX_PROBE(2, true); break;
    default: DSX_PROBE(3, true); break;
  }
#undef DSX_PROBE
  const int64_t flops_per_mfma[4] = {2ll * 32 * 32 * 16, 2ll * 32 * 32 * 64, 2ll * 16 * 16 * 32, 2ll * 16 * 16 * 128};
  const int64_t mfmas_per_iter = (kind & 3) >= 2 ? 8 : 4;  // the small shapes run eight independent accumulators
  if (flops_out) *flops_out = (int64_t)workgroups * 4 * iters * mfmas_per_iter * flops_per_mfma[kind & 3];
  return hipGetLastError() == hipSuccess ? DSX_OK : DSX_ELAUNCH;
}
