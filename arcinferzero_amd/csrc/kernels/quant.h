// The per-block int8 activation quantizer shared by the kernels that produce matmul inputs.
// Per block of 32 (act32) or 256 values (reference zero/kernels/ops.cl:38-72, src/quants.h:626-643):
//   amax = max |v|;  inv = amax > 0 ? 127 / amax : 0;  q = rte(v * inv) (one f32 multiply);  scale = amax / 127.
// A thread holds 16 consecutive values; the 2 (act32) or 16 threads of a block are neighbouring lanes.
#pragma once
#include "common.h"

__device__ inline float block_amax(const float* v, int act32) {
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[i]));
  amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
  if (!act32) {
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 8, 64));
  }
  return amax;
}

// Quantizes v[16] (the 16 values of lane16 in its row's superblock); returns the packed int8 and their sum.  With
// res, also what the int8 values miss: res[i] = v[i] - (float)q * (amax / 127) (reference zero/kernels/ops.cl:49-59,
// the two-pass mode's residual; the product and the difference are rounded one after the other).
__device__ inline void quant16(const float* v, float amax, uint4& pk, int& sum, float* res = nullptr) {
#pragma clang fp contract(off)  // (no fused multiply-add below: v * inv and q * scale are rounded on their own)
  const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
  const float sc = amax / 127.0f;
  uint32_t w[4] = {0, 0, 0, 0};
  sum = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float p = __fmul_rn(v[i], inv);
    const int q = __float2int_rn(p);
    sum += q;
    w[i >> 2] |= (uint32_t)(q & 0xFF) << (8 * (i & 3));
    if (res) {  // (plain operators: under the pragma above they carry no licence to fuse)
      const float qs = (float)q * sc;
      res[i] = v[i] - qs;
    }
  }
  pk = make_uint4(w[0], w[1], w[2], w[3]);
}

