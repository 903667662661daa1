// One row of per-row dynamic quantisation to OCP fp8 e4m3, by one wavefront.
#pragma once
#include "fr_common.h"

namespace fr {

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> { typedef bf16x8 type; };
template <> struct Vec8<f16_t> { typedef f16x8 type; };

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, partner_f32<1>(v));
  v = fmaxf(v, partner_f32<2>(v));
  v = fmaxf(v, partner_f32<4>(v));
  v = fmaxf(v, partner_f32<8>(v));
  v = fmaxf(v, partner_f32<16>(v));
  v = fmaxf(v, partner_f32<32>(v));
  return v;
}

__device__ __forceinline__ unsigned pack4(float a, float b, float c, float d) {
  int w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return static_cast<unsigned>(w);
}

// Pass 1 reduces max|x| across the row (16-byte loads, cross-lane butterfly), scale = amax/448 (1 for an
// all-zero row); pass 2 re-reads the row (L2-resident) and converts x/scale with v_cvt_pk_fp8_f32 (round
// to nearest even), 16 codes per 16-byte store.  xr: the row's K elements; qr: its K codes; *scale_out: its scale.
template <typename T>
__device__ __forceinline__ void quant_row(const T* __restrict__ xr, int K, unsigned char* __restrict__ qr,
                                          float* __restrict__ scale_out, int lane) {
  typedef typename Vec8<T>::type vec8;
  float amax = 0.f;
  for (int k = lane * 8; k < K; k += kWave * 8) {
    const vec8 v = *reinterpret_cast<const vec8*>(xr + k);
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(static_cast<float>(v[i])));
  }
  amax = wave_max(amax);
  const float s = amax > 0.f ? amax / 448.f : 1.f;
  if (lane == 0) *scale_out = s;
  // x / s for every element of the row.  With y = RN(1/s), q = RN(x*y), r = RN(x - s*q) (one
  // FMA), RN(q + r*y) (Markstein's correction step) equals the IEEE quotient as long as nothing
  // leaves the normal range - no mismatch against exact rational arithmetic on 7e5 sampled
  // bf16/fp16 pairs.  Rows with 2^-40 <= max|x| <= 2^40 take this 3-instruction form (there an
  // element below 2^-70, whose r could be subnormal, has |x/s| < 2^-21 and encodes as zero either
  // way); any other row the IEEE division, 10 instructions per element.
  const bool fast = amax >= 0x1p-40f && amax <= 0x1p40f;
  const float y = 1.f / s;
  auto quot = [&](float x) {
    if (fast) {
      const float q0 = x * y;
      const float r = __builtin_fmaf(-s, q0, x);
      return __builtin_fmaf(r, y, q0);
    }
    return x / s;
  };
  for (int k = lane * 16; k < K; k += kWave * 16) {
    const vec8 v0 = *reinterpret_cast<const vec8*>(xr + k);
    const vec8 v1 = *reinterpret_cast<const vec8*>(xr + k + 8);
    float f[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      f[i] = fminf(fmaxf(quot(static_cast<float>(v0[i])), -448.f), 448.f);
      f[8 + i] = fminf(fmaxf(quot(static_cast<float>(v1[i])), -448.f), 448.f);
    }
    u32x4_t o;
    o.x = pack4(f[0], f[1], f[2], f[3]);
    o.y = pack4(f[4], f[5], f[6], f[7]);
    o.z = pack4(f[8], f[9], f[10], f[11]);
    o.w = pack4(f[12], f[13], f[14], f[15]);
    *reinterpret_cast<u32x4_t*>(qr + k) = o;
  }
}

// The same result from one read of the row, by a workgroup of NW wavefronts: the row's K <= 512 * NW * NC
// elements stay in registers (NC 16-byte chunks per thread, chunk c * 64 * NW + tid: every load and every
// 8-byte store of a wavefront is contiguous) between the reduction and the conversion; all NC loads of a
// thread are in flight at once, and the wavefronts' maxima meet in `red` (NW floats of LDS).
template <typename T, int NC, int NW>
__device__ __forceinline__ void quant_row_block(const T* __restrict__ xr, int K, unsigned char* __restrict__ qr,
                                                float* __restrict__ scale_out, int tid, float* red) {
  typedef typename Vec8<T>::type vec8;
  vec8 v[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int k = (c * kWave * NW + tid) * 8;
    if (k < K) v[c] = *reinterpret_cast<const vec8*>(xr + k);
    else v[c] = vec8{0, 0, 0, 0, 0, 0, 0, 0};
  }
  float amax = 0.f;
#pragma unroll
  for (int c = 0; c < NC; ++c)
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(static_cast<float>(v[c][i])));
  amax = wave_max(amax);
  if (tid % kWave == 0) red[tid / kWave] = amax;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < NW; ++w) amax = fmaxf(amax, red[w]);
  const float s = amax > 0.f ? amax / 448.f : 1.f;
  if (tid == 0) *scale_out = s;
  const bool fast = amax >= 0x1p-40f && amax <= 0x1p40f;  // see quant_row
  const float y = 1.f / s;
  auto quot = [&](float x) {
    if (fast) {
      const float q0 = x * y;
      const float r = __builtin_fmaf(-s, q0, x);
      return __builtin_fmaf(r, y, q0);
    }
    return x / s;
  };
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int k = (c * kWave * NW + tid) * 8;
    float f[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = fminf(fmaxf(quot(static_cast<float>(v[c][i])), -448.f), 448.f);
    uint2 o;
    o.x = pack4(f[0], f[1], f[2], f[3]);
    o.y = pack4(f[4], f[5], f[6], f[7]);
    if (k < K) *reinterpret_cast<uint2*>(qr + k) = o;
  }
}

}  // namespace fr
