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
  const unsigned vkey = float_key(v[0] + 0.f);  // + 0.f: -0 and +0 are the same value
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

// Many experts: a group of only G lanes owns a token and every lane keeps NV vectors of 4
// consecutive logits, vector j of lane g holding experts 4*(G*j + g) .. 4*(G*j + g) + 3, so
// the G lanes read 4*G consecutive logits of the token per load and a wavefront gates 64/G
// tokens at once: the cross-lane rounds (the cost of the one-logit-per-lane form, a wavefront
// instruction per step per token) shrink to log2(G) steps shared by 64/G tokens.  Inside a
// lane expert indices rise with the slot number, across lanes ties go to the lower index,
// so the order is still (value descending, index ascending).  load4(e0) returns logits
// e0..e0+3; E must be a multiple of 4.
constexpr int kBlockedSlots = 4;  // result slots per lane: topk <= kBlockedSlots * G

template <int G, int NV, typename Load4>
__device__ __forceinline__ void gate_token_blocked(Load4 load4, bool live, int E, int topk, int renorm,
                                                   float* __restrict__ w_row, int32_t* __restrict__ id_row) {
  constexpr int VPL = 4 * NV;
  static_assert(G <= 16, "the all-reduce uses the in-row DPP steps only");
  const int g = threadIdx.x % G;
  float v[VPL];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int e0 = 4 * (G * j + g);
    f32x4 t = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    if (live && e0 < E) t = load4(e0);
#pragma unroll
    for (int c = 0; c < 4; ++c) v[4 * j + c] = t[c];
  }
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

  // Order keys of this lane's logits (0 = not a candidate).  Inside the lane a strict
  // "greater" scan keeps the lowest slot, i.e. the lowest expert index, among equal keys.
  unsigned k[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = 4 * (G * (i / 4) + g) + (i % 4);
    k[i] = (e < E) ? float_key(v[i] + 0.f) : 0u;  // + 0.f: -0 and +0 are the same value
  }
  float sel_v[kBlockedSlots];
  int sel_i[kBlockedSlots];
#pragma unroll
  for (int i = 0; i < kBlockedSlots; ++i) {
    sel_v[i] = -INFINITY;
    sel_i[i] = 0;
  }
  int last = -1;  // slot this lane gave away in the previous round
  float sel_sum = 0.f;
  for (int r = 0; r < topk; ++r) {
    unsigned bk = 0u;
    int bs = 0;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      if (i == last) k[i] = 0u;
      if (k[i] > bk) {
        bk = k[i];
        bs = i;
      }
    }
    int be = 4 * (G * (bs >> 2) + g) + (bs & 3);
    // all-reduce over the group: larger key wins, equal keys go to the lower expert index
    auto step = [&](auto tag) {
      constexpr int S = decltype(tag)::value;
      const unsigned ok = static_cast<unsigned>(partner_i32<S>(static_cast<int>(bk)));
      const int oe = partner_i32<S>(be);
      if (ok > bk || (ok == bk && oe < be)) {
        bk = ok;
        be = oe;
      }
    };
    if constexpr (G > 1) step(std::integral_constant<int, 1>{});
    if constexpr (G > 2) step(std::integral_constant<int, 2>{});
    if constexpr (G > 4) step(std::integral_constant<int, 4>{});
    if constexpr (G > 8) step(std::integral_constant<int, 8>{});
    last = ((be >> 2) % G == g) ? (4 * (be / (4 * G)) + (be & 3)) : -1;
    const float bv = key_float(bk);
    sel_sum += __expf(bv - m);
#pragma unroll
    for (int sl = 0; sl < kBlockedSlots; ++sl) {
      if (r == sl * G + g) {
        sel_v[sl] = bv;
        sel_i[sl] = be;
      }
    }
  }
  const float denom = renorm ? sel_sum : s;
  if (live) {
#pragma unroll
    for (int sl = 0; sl < kBlockedSlots; ++sl) {
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
