// The routing of one token by one wave, shared by the kernels that route (reference zero/kernels/moe.cl:50-109): the NU
// largest of NE logits (ties: the lower expert), p = exp(l - max), weights p / sum of the selected p.  Lane k < NU
// returns the k-th choice and its weight.  NE <= 512.
#pragma once
#include "common.h"

#define ROUTE_PER_LANE 8

// The better of two (value, expert) candidates: the larger value, the lower expert among equal values.
__device__ inline void route_better(float& bv, int& bi, float ov, int oi) {
  if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}
// Wave arg-max of (bv, bi), the result in every lane: four steps inside each row of 16 lanes in the vector ALU (quad
// swaps, then the row's mirrors: lanes that have met hold the same candidate, so a mirrored lane brings the other
// group's), then the four rows' candidates read as scalars.  (Through the LDS crossbar the six dependent exchanges of
// a round were most of a routing kernel's time.)
__device__ inline void route_wave_best(float& bv, int& bi) {
#define ROUTE_STEP(CTRL)                                                                             \
  route_better(bv, bi, __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(bv), CTRL, 0xF, 0xF, true)), \
               __builtin_amdgcn_mov_dpp(bi, CTRL, 0xF, 0xF, true));
  ROUTE_STEP(0xB1) ROUTE_STEP(0x4E) ROUTE_STEP(0x141) ROUTE_STEP(0x140)
#undef ROUTE_STEP
  float rv[4];
  int ri[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    rv[r] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(bv), 16 * r));
    ri[r] = __builtin_amdgcn_readlane(bi, 16 * r);
  }
  bv = rv[0];
  bi = ri[0];
#pragma unroll
  for (int r = 1; r < 4; ++r) route_better(bv, bi, rv[r], ri[r]);
}

// The reference's routing variants (zero/kernels/moe.cl:17-46), chosen per launch: escale (its -DESCALE, Gemma 4) -- each
// chosen expert's weight times escale[e] after the normalization; ebias (its -DROUTE_DS, DeepSeek-V4.1) -- the score is
// s = sqrt(softplus(logit)), experts are chosen by s + ebias[e], and the weights are s / (sum of the chosen s + 1e-20) *
// rscale.  Both null: the softmax routing.
struct RouteVariant {
  const float* escale = nullptr;
  const float* ebias = nullptr;
  float rscale = 1.0f;
};
__device__ inline float route_ds_sp(float g) { return sqrtf(g > 20.0f ? g + log1pf(expf(-g)) : log1pf(expf(g))); }

template <int PL>
__device__ inline void route_one_token_pl(const float* __restrict__ lg, int NE, int NU, int lane, int& sel, float& wt,
                                          const RouteVariant rv = RouteVariant()) {
  float v[PL];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < PL; ++i) {
    const int e = i * 64 + lane;
    v[i] = e < NE ? (rv.ebias ? route_ds_sp(lg[e]) + rv.ebias[e] : lg[e]) : -INFINITY;
    mx = fmaxf(mx, v[i]);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
  float sum = 0.0f, myp = 0.0f;
  int mysel = 0;
  for (int k = 0; k < NU; ++k) {
    float bv = -INFINITY;
    int bi = NE;
#pragma unroll
    for (int i = 0; i < PL; ++i)
      if (v[i] > bv) { bv = v[i]; bi = i * 64 + lane; }
    route_wave_best(bv, bi);
#pragma unroll
    for (int i = 0; i < PL; ++i)
      if (i * 64 + lane == bi) v[i] = -INFINITY;
    const int sk = min(bi, NE - 1);  // (a row of NaN picks no lane: keep the index inside the tables)
    const float p = rv.ebias ? route_ds_sp(lg[sk]) : expf(bv - mx);
    sum += p;
    if (lane == k) { mysel = sk; myp = p; }
  }
  sel = mysel;
  wt = rv.ebias ? myp / (sum + 1e-20f) * rv.rscale : myp / sum;
  if (rv.escale) wt *= rv.escale[mysel];
}

// (two logits a lane serve up to 128 experts, the common case; the same steps either way)
__device__ inline void route_one_token(const float* __restrict__ lg, int NE, int NU, int lane, int& sel, float& wt,
                                       const RouteVariant rv = RouteVariant()) {
  if (NE <= 128) route_one_token_pl<2>(lg, NE, NU, lane, sel, wt, rv);
  else route_one_token_pl<ROUTE_PER_LANE>(lg, NE, NU, lane, sel, wt, rv);
}
// The shared expert's gate of a token (moe.cl:40, 46): sigmoid of the logit past the experts' when the row holds one;
// 1 with the -DROUTE_DS routing.
__device__ inline float route_sgate(const float* __restrict__ lg, int NE, bool has_gate, const RouteVariant rv) {
  return rv.ebias ? 1.0f : has_gate ? 1.0f / (1.0f + expf(-lg[NE])) : 0.0f;
}
