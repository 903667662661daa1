// Measurement aid: a pure MFMA stream on caller-provided operand bits, to read the rate and the shader
// clock the part sustains under MFMA load (it lowers its clock to hold a power budget; the figure depends
// on the MFMA shape, on how many wavefronts share a SIMD and on the operand data).
#include "fr_common.h"

namespace fr {
namespace {
typedef unsigned int u32x4p __attribute__((ext_vector_type(4)));

// SHAPE 32: v_mfma_f32_32x32x16_bf16, NA accumulators of 16 registers; SHAPE 16: v_mfma_f32_16x16x32_bf16, NA of 4.
// One workgroup per CU, NT / 256 wavefronts per SIMD; operands: 4096 x 16 bytes.
template <int SHAPE, int NA, int NT>
__global__ __launch_bounds__(NT) void mfma_stream_kernel(const u32x4p* __restrict__ src, float* __restrict__ sink,
                                                         long long* __restrict__ counts, int iters) {
  typedef typename std::conditional<SHAPE == 32, f32x16, f32x4>::type acc_t;
  constexpr int NF = 8, NR = SHAPE == 32 ? 16 : 4;
  u32x4p fa[NF], fb[NF];
#pragma unroll
  for (int i = 0; i < NF; ++i) {
    fa[i] = src[(threadIdx.x * 7 + i * 131) & 4095];
    fb[i] = src[(threadIdx.x * 13 + i * 977 + 5) & 4095];
  }
  acc_t acc[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i)
#pragma unroll
    for (int r = 0; r < NR; ++r) acc[i][r] = 0.f;
  const long long t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < NA; ++m) {
      if constexpr (SHAPE == 32)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[(m / 4) % NF]), __builtin_bit_cast(bf16x8, fb[m % 4 + (m / 16) % 2 * 4]), acc[m], 0, 0, 0);
      else
        acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fa[(m / 8) % NF]), __builtin_bit_cast(bf16x8, fb[m % 8]), acc[m], 0, 0, 0);
    }
  }
  const long long t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NA; ++i) s += acc[i][1];
  sink[blockIdx.x * NT + threadIdx.x] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    counts[0] = t1 - t0;  // shader clock cycles
    counts[1] = r1 - r0;  // ticks of the constant 100 MHz counter
  }
}
}  // namespace
}  // namespace fr

using namespace fr;

extern "C" int fr_probe_mfma_stream(int shape, int waves_per_simd, int iters, const void* operands, float* sink,
                                    int64_t* counts, void* stream) {
  FR_REQUIRE((shape == 16 || shape == 32) && (waves_per_simd == 1 || waves_per_simd == 2) && iters >= 1, FR_E_SHAPE,
             "fr_probe_mfma_stream: shape=%d (16 or 32), waves_per_simd=%d (1 or 2), iters=%d", shape, waves_per_simd, iters);
  FR_REQUIRE(operands && sink && counts, FR_E_NULL, "fr_probe_mfma_stream: null pointer");
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
    return fail(FR_E_NO_DEVICE, "fr_probe_mfma_stream: no device");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const u32x4p* src = static_cast<const u32x4p*>(operands);
  long long* cnt = reinterpret_cast<long long*>(counts);
  // 256 accumulator registers per lane with one wavefront per SIMD, 128 each with two
  if (shape == 32 && waves_per_simd == 1) hipLaunchKernelGGL((mfma_stream_kernel<32, 16, 256>), dim3(cus), dim3(256), 0, st, src, sink, cnt, iters);
  else if (shape == 32) hipLaunchKernelGGL((mfma_stream_kernel<32, 8, 512>), dim3(cus), dim3(512), 0, st, src, sink, cnt, iters);
  else if (waves_per_simd == 1) hipLaunchKernelGGL((mfma_stream_kernel<16, 64, 256>), dim3(cus), dim3(256), 0, st, src, sink, cnt, iters);
  else hipLaunchKernelGGL((mfma_stream_kernel<16, 32, 512>), dim3(cus), dim3(512), 0, st, src, sink, cnt, iters);
  return check_launch("mfma_stream_kernel");
}
