// Gating core shared by the gating kernels and the fused small-batch routing kernel:
// cross-lane reductions over a group of G lanes and gate_token(), the top-k gating of one
// token by one lane group.
#pragma once
#include "fr_common.h"

#include <float.h>
#include <limits.h>

#include <type_traits>

namespace fr {
namespace {

__device__ __forceinline__ bool better(float av, int ai, float bv, int bi) {
  return av > bv || (av == bv && ai < bi);
}

// max over the group, returned in every lane: DPP steps inside a row of 16 lanes,
// then the (uniform per row) row maxima are read out as scalars and combined
template <int G>
__device__ __forceinline__ float group_max(float v) {
  if constexpr (G > 1) v = fmaxf(v, partner_f32<1>(v));
  if constexpr (G > 2) v = fmaxf(v, partner_f32<2>(v));
  if constexpr (G > 4) v = fmaxf(v, partner_f32<4>(v));
  if constexpr (G > 8) v = fmaxf(v, partner_f32<8>(v));
  if constexpr (G > 16) {
    const int bits = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(bits, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(bits, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
    if constexpr (G == 32) v = (threadIdx.x & 32) ? fmaxf(r2, r3) : fmaxf(r0, r1);
    else v = fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
  }
  return v;
}

// sum over the group, same scheme (every lane adds the same numbers in the same order)
template <int G>
__device__ __forceinline__ float group_sum(float v) {
  if constexpr (G > 1) v += partner_f32<1>(v);
  if constexpr (G > 2) v += partner_f32<2>(v);
  if constexpr (G > 4) v += partner_f32<4>(v);
  if constexpr (G > 8) v += partner_f32<8>(v);
  if constexpr (G > 16) {
    const int bits = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(bits, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(bits, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
    if constexpr (G == 32) v = (threadIdx.x & 32) ? (r2 + r3) : (r0 + r1);
    else v = (r0 + r1) + (r2 + r3);
  }
  return v;
}

// Order-preserving map fp32 -> uint32 (larger float <=> larger key; every real value,
// -inf included, maps above 0, which serves as "not a candidate").
__device__ __forceinline__ unsigned float_key(float v) {
  const unsigned b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_float(unsigned k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}
// unsigned max over the group, in every lane (integer max needs no NaN canonicalisation,
// so the DPP moves fold into v_max_u32; rows are combined on the scalar unit)
template <int G>
__device__ __forceinline__ unsigned group_max_key(unsigned k) {
  if constexpr (G > 1) k = max(k, static_cast<unsigned>(partner_i32<1>(static_cast<int>(k))));
  if constexpr (G > 2) k = max(k, static_cast<unsigned>(partner_i32<2>(static_cast<int>(k))));
  if constexpr (G > 4) k = max(k, static_cast<unsigned>(partner_i32<4>(static_cast<int>(k))));
  if constexpr (G > 8) k = max(k, static_cast<unsigned>(partner_i32<8>(static_cast<int>(k))));
  if constexpr (G > 16) {
    const unsigned r0 = __builtin_amdgcn_readlane(static_cast<int>(k), 0);
    const unsigned r1 = __builtin_amdgcn_readlane(static_cast<int>(k), 16);
    const unsigned r2 = __builtin_amdgcn_readlane(static_cast<int>(k), 32);
    const unsigned r3 = __builtin_amdgcn_readlane(static_cast<int>(k), 48);
    if constexpr (G == 32) k = (threadIdx.x & 32) ? max(r2, r3) : max(r0, r1);
    else k = max(max(r0, r1), max(r2, r3));
  }
  return k;
}

// Cross-lane merge of per-lane online-softmax states (m = running max, s = sum of
// exp(x - m)): one max reduction, one rescale, one sum reduction.
template <int G>
__device__ __forceinline__ void group_online_softmax(float& m, float& s) {
  const float gm = group_max<G>(m);
  s = group_sum<G>((m == -INFINITY) ? 0.f : s * __expf(m - gm));
  m = gm;
}

template <int G>
__device__ __forceinline__ void group_argmax(float& v, int& i) {
  auto step = [&](auto tag) {
    constexpr int S = decltype(tag)::value;
    const float ov = partner_f32<S>(v);
    const int oi = partner_i32<S>(i);
    if (better(ov, oi, v, i)) {
      v = ov;
      i = oi;
    }
  };
  if constexpr (G > 1) step(std::integral_constant<int, 1>{});
  if constexpr (G > 2) step(std::integral_constant<int, 2>{});
  if constexpr (G > 4) step(std::integral_constant<int, 4>{});
  if constexpr (G > 8) step(std::integral_constant<int, 8>{});
  if constexpr (G > 16) step(std::integral_constant<int, 16>{});
  if constexpr (G > 32) step(std::integral_constant<int, 32>{});
}

constexpr int kGateThreads = 256;

// Gating of one token by a group of G lanes.  `load(e)` returns logit e as fp32;
// every lane of the wavefront must call this (dead groups pass live = false).
template <int G, int VPL, typename Load>
__device__ __forceinline__ void gate_token(Load load, bool live, int E, int topk, int renorm,
                                           float* __restrict__ w_row, int32_t* __restrict__ id_row) {
  const int g = threadIdx.x % G;
  float v[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = g + i * G;
    v[i] = (live && e < E) ? load(e) : -INFINITY;
  }

  // online softmax over this lane's values (running max, rescaled running sum),
  // then merged across the group
  float m = v[0];
  float s = (v[0] == -INFINITY) ? 0.f : 1.f;
#pragma unroll
  for (int i = 1; i < VPL; ++i) {
    if (v[i] == -INFINITY) continue;
    const float mn = fmaxf(m, v[i]);
    s = (m == -INFINITY ? 0.f : s * __expf(m - mn)) + __expf(v[i] - mn);
    m = mn;
  }
  group_online_softmax<G>(m, s);

  float sel_v[VPL];
  int sel_i[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    sel_v[i] = -INFINITY;
    sel_i[i] = 0;
  }
  unsigned taken = 0;
  float sel_sum = 0.f;
  const unsigned vkey = float_key(v[0]);
  for (int r = 0; r < topk; ++r) {
    float bv;
    int bi;
    if constexpr (VPL == 1) {
      // one logit per lane, lane order = expert order: the winner is the group max and,
      // among lanes holding it, the lowest lane (= lowest expert index) of a ballot
      const unsigned key = (g < E && !taken) ? vkey : 0u;
      const unsigned top = group_max_key<G>(key);
      bv = key_float(top);
      unsigned long long hit = __ballot(key == top);
      if constexpr (G < 64) hit = (hit >> (threadIdx.x & 63 & ~(G - 1))) & ((1ull << G) - 1ull);
      bi = __ffsll(hit) - 1;
      if (bi == g) taken = 1u;
    } else {
      bv = -INFINITY;
      bi = INT_MAX;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int e = g + i * G;
        if (e < E && !((taken >> i) & 1u) && better(v[i], e, bv, bi)) {
          bv = v[i];
          bi = e;
        }
      }
      group_argmax<G>(bv, bi);
      if (bi % G == g) taken |= 1u << (bi / G);
    }
    sel_sum += __expf(bv - m);
#pragma unroll
    for (int sl = 0; sl < VPL; ++sl) {
      if (r == sl * G + g) {
        sel_v[sl] = bv;
        sel_i[sl] = bi;
      }
    }
  }

  const float denom = renorm ? sel_sum : s;
  if (live) {
#pragma unroll
    for (int sl = 0; sl < VPL; ++sl) {
      const int r = sl * G + g;
      if (r < topk) {
        w_row[r] = __expf(sel_v[sl] - m) / denom;
        id_row[r] = sel_i[sl];
      }
    }
  }
}

}  // namespace
}  // namespace fr
