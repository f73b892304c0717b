// "ops" module: the activation quantizer that feeds every block-quantized matmul, alone and fused into the two
// producers the matmul path uses (RMS norm, SwiGLU).
//
// Arithmetic per block of 32 (act32) or 256 values, as the reference's quant_store16 (zero/kernels/ops.cl:38-72,
// CPU twin src/quants.h:626-643):  amax = max |v|;  inv = amax > 0 ? 127 / amax : 0;  q = rte(v * inv) (one f32
// multiply, then round to nearest even);  scale = amax / 127 (a true division);  absum = int16 sum of each 16 q.
// Layouts: aq [M][K] int8, asc [K/32][M] (or [K/256][M]) f32, absum [K/16][M] int16.  Rows m >= T are written as
// zeros with scale 0 (the padding rows of a prompt chunk).
//
// Two-pass mode (reference zero/kernels/ops.cl:73-101, its -DQ2_AQ / -DQ2_SC / -DQ2_AB; here the three offsets are
// trailing arguments, 0 = off): the residual v - q * scale of every value is quantized the same way into the same
// layouts q2_aq bytes / q2_sc floats / q2_ab shorts further on in the three buffers, for a second matmul pass that
// accumulates into the first one's output.
//
// Mapping: a work-group of 256 threads takes one superblock (256 values) of 64 token rows.  Thread t holds 16
// consecutive values of one row (16 threads = one row's superblock, read as one contiguous KiB); the two threads of a
// 32-block exchange their maxima with one cross-lane move.  Scales and sums go through LDS so that they leave as
// runs of 64 consecutive tokens (the token-minor layout the matmuls read).
#include "quant.h"

// Shared tail of the row kernels: stores one tile's scales and sums token-minor.
struct QuantTile {
  float asc[8][64];
  short sum[16][64];
};

__device__ inline void store_tile_scales(const QuantTile& lds, int s, int m0, int M, int act32, float* asc,
                                         short* absum) {
  const int t = threadIdx.x;
  if (act32) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = t + 256 * i, b = idx >> 6, r = idx & 63;
      if (m0 + r < M) asc[((size_t)s * 8 + b) * M + m0 + r] = lds.asc[b][r];
    }
  } else if (t < 64) {
    if (m0 + t < M) asc[(size_t)s * M + m0 + t] = lds.asc[0][t];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = t + 256 * i, h = idx >> 6, r = idx & 63;
    if (m0 + r < M) absum[((size_t)s * 16 + h) * M + m0 + r] = lds.sum[h][r];
  }
}

// quant_rows: x [T][ldx] f32 -> aq / asc / absum for M rows (rows >= T zero).  grid (K/256, ceil(M/64)), local 256.
extern "C" __global__ __launch_bounds__(256) void quant_rows(const float* __restrict__ x, int ldx, int K, int M, int T,
                                                             signed char* __restrict__ aq, float* __restrict__ asc,
                                                             short* __restrict__ absum, int act32, int q2_aq, int q2_sc,
                                                             int q2_ab) {
  __shared__ QuantTile lds, lds2;
  const int s = blockIdx.x, m0 = blockIdx.y * 64;
  const int lane16 = threadIdx.x & 15, rg = threadIdx.x >> 4;
#pragma unroll 1
  for (int p = 0; p < 4; ++p) {
    const int r = p * 16 + rg, m = m0 + r;
    float v[16];
    if (m < T) {
      const float4* src = (const float4*)(x + (size_t)m * ldx + s * 256 + 16 * lane16);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 f = src[i];
        v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = 0.0f;
    }
    const float amax = block_amax(v, act32);
    uint4 pk;
    int sum;
    float res[16];
    quant16(v, amax, pk, sum, q2_aq ? res : nullptr);
    if (m < M) *(uint4*)(aq + (size_t)m * K + s * 256 + 16 * lane16) = pk;
    lds.sum[lane16][r] = (short)sum;
    if (act32) {
      if ((lane16 & 1) == 0) lds.asc[lane16 >> 1][r] = amax / 127.0f;
    } else if (lane16 == 0) {
      lds.asc[0][r] = amax / 127.0f;
    }
    if (q2_aq) {  // (the same for the whole launch)
      const float rmax = block_amax(res, act32);
      quant16(res, rmax, pk, sum);
      if (m < M) *(uint4*)(aq + q2_aq + (size_t)m * K + s * 256 + 16 * lane16) = pk;
      lds2.sum[lane16][r] = (short)sum;
      if (act32) {
        if ((lane16 & 1) == 0) lds2.asc[lane16 >> 1][r] = rmax / 127.0f;
      } else if (lane16 == 0) {
        lds2.asc[0][r] = rmax / 127.0f;
      }
    }
  }
  __syncthreads();
  store_tile_scales(lds, s, m0, M, act32, asc, absum);
  if (q2_aq) store_tile_scales(lds2, s, m0, M, act32, asc + q2_sc, absum + q2_ab);
}

// ---- the two fused producers.  A work-group of 256 threads per row (or several along x, each taking a share of the
// row's superblocks: the launch for a pass of 1-8 tokens, zero/engine.h:1404-1412); 16 threads per superblock, thread
// = 16 consecutive values, so a wave works on 4 superblocks at a time.  Scales and sums are stored straight into the
// token-minor layouts (one element per block and row).
__device__ inline void store_row_quant1(const float* v, int s, int lane16, int m, int M, int K, int act32,
                                        signed char* __restrict__ aq, float* __restrict__ asc, short* __restrict__ absum,
                                        float* res) {
  const float amax = block_amax(v, act32);
  uint4 pk;
  int sum;
  quant16(v, amax, pk, sum, res);
  *(uint4*)(aq + (size_t)m * K + s * 256 + 16 * lane16) = pk;
  absum[((size_t)s * 16 + lane16) * M + m] = (short)sum;
  if (act32) {
    if ((lane16 & 1) == 0) asc[((size_t)s * 8 + (lane16 >> 1)) * M + m] = amax / 127.0f;
  } else if (lane16 == 0) {
    asc[(size_t)s * M + m] = amax / 127.0f;
  }
}
// (q2_aq != 0: the two-pass mode's residual too, at its offsets in the same buffers)
__device__ inline void store_row_quant(const float* v, int s, int lane16, int m, int M, int K, int act32,
                                       signed char* __restrict__ aq, float* __restrict__ asc, short* __restrict__ absum,
                                       int q2_aq, int q2_sc, int q2_ab) {
  if (!q2_aq) {
    store_row_quant1(v, s, lane16, m, M, K, act32, aq, asc, absum, nullptr);
  } else {
    float res[16];
    store_row_quant1(v, s, lane16, m, M, K, act32, aq, asc, absum, res);
    store_row_quant1(res, s, lane16, m, M, K, act32, aq + q2_aq, asc + q2_sc, absum + q2_ab, nullptr);
  }
}

// Sum over the work-group, the same value in every thread, in a fixed order (so every work-group that sums the same
// row gets the same bits).
__device__ inline float group_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  const float r = (red[0] + red[1]) + (red[2] + red[3]);
  __syncthreads();
  return r;
}

// rmsnorm_quant: y = x[row_off + m] * rsqrt(mean(x^2) + eps) * w, quantized for the next matmul, rows m >= M_valid as
// zeros; with write_h also stored as f32 in hout [M][K] (reference zero/kernels/ops.cl:107-141, same arguments).
// grid (256 * G, rows), local (256, 1).
extern "C" __global__ __launch_bounds__(256) void rmsnorm_quant(const float* __restrict__ x, int row_off,
                                                                const float* __restrict__ w, int K, int M, int M_valid,
                                                                float eps, signed char* __restrict__ aq,
                                                                float* __restrict__ asc, short* __restrict__ absum,
                                                                float* __restrict__ hout, int write_h, int act32,
                                                                int q2_aq, int q2_sc, int q2_ab) {
  __shared__ float red[4];
  const int m = blockIdx.y;
  const bool valid = m < M_valid;
  const float* xr = x + (size_t)(m + row_off) * K;
  const int lane16 = threadIdx.x & 15, sub = threadIdx.x >> 4;
  constexpr int MAXU = 5;  // superblocks a thread can hold: rows of up to 16 * 5 * 256 = 20480 values
  if (gridDim.x == 1 && K <= 16 * MAXU * 256) {
    // One work-group per row: the row stays in registers between the sum of squares and the quantization (a thread
    // holds its 16 values of superblocks sub, sub + 16, ...), so x is read once, every load of the row in flight at once.
    const int nsb = K >> 8;
    float4 xv[MAXU][4];
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      const int sb = sub + 16 * u;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        xv[u][i] = valid && sb < nsb ? *(const float4*)(xr + sb * 256 + 16 * lane16 + 4 * i) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    float ss = 0.0f;
#pragma unroll
    for (int u = 0; u < MAXU; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ss += xv[u][i].x * xv[u][i].x;
        ss += xv[u][i].y * xv[u][i].y;
        ss += xv[u][i].z * xv[u][i].z;
        ss += xv[u][i].w * xv[u][i].w;
      }
    ss = group_sum(ss, red);
    const float r = rsqrtf(ss / (float)K + eps);
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      const int sb = sub + 16 * u;
      if (sb >= nsb) break;  // (the same for the 16 threads of a superblock)
      const int base = sb * 256 + 16 * lane16;
      float v[16];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 f = xv[u][i], g = *(const float4*)(w + base + 4 * i);
        v[4 * i] = f.x * r * g.x; v[4 * i + 1] = f.y * r * g.y; v[4 * i + 2] = f.z * r * g.z; v[4 * i + 3] = f.w * r * g.w;
      }
      if (write_h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          *(float4*)(hout + (size_t)m * K + base + 4 * i) = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
      store_row_quant(v, sb, lane16, m, M, K, act32, aq, asc, absum, q2_aq, q2_sc, q2_ab);
    }
    return;
  }
  float ss = 0.0f;
  if (valid)
    for (int i = threadIdx.x * 4; i < K; i += 1024) {
      const float4 f = *(const float4*)(xr + i);
      ss += f.x * f.x;
      ss += f.y * f.y;
      ss += f.z * f.z;
      ss += f.w * f.w;
    }
  ss = group_sum(ss, red);
  const float r = rsqrtf(ss / (float)K + eps);
  for (int s = blockIdx.x * 16 + sub; s < K / 256; s += 16 * gridDim.x) {
    const int base = s * 256 + 16 * lane16;
    float v[16];
    if (valid) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 f = *(const float4*)(xr + base + 4 * i), g = *(const float4*)(w + base + 4 * i);
        v[4 * i] = f.x * r * g.x; v[4 * i + 1] = f.y * r * g.y; v[4 * i + 2] = f.z * r * g.z; v[4 * i + 3] = f.w * r * g.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = 0.0f;
    }
    if (write_h)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *(float4*)(hout + (size_t)m * K + base + 4 * i) = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    store_row_quant(v, s, lane16, m, M, K, act32, aq, asc, absum, q2_aq, q2_sc, q2_ab);
  }
}

// add_norm_quant: x[m] = (x[m] + rmsnorm(t[m]) * w) * s in place (Gemma's post-norm residual add with the layer's
// output scale), then the next matmul's input from the new row: rmsnorm(x[m]) * w2, or the row itself with w2_norm = 0,
// quantized (reference zero/kernels/ops_attn_g.cl:616-667, same arguments plus M_valid: rows from M_valid on are
// written as zeros where the reference launches the valid rows only).  Both sums of squares run in a fixed order.  A
// thread reads back the values it has just stored to x itself, which the memory model orders.  grid (256, rows),
// local (256, 1).
extern "C" __global__ __launch_bounds__(256) void add_norm_quant(float* __restrict__ x, const float* __restrict__ t,
                                                                 const float* __restrict__ w, int K, float eps, float s,
                                                                 const float* __restrict__ w2, int w2_norm, int M,
                                                                 signed char* __restrict__ aq, float* __restrict__ asc,
                                                                 short* __restrict__ absum, int act32, int M_valid,
                                                                 int q2_aq, int q2_sc, int q2_ab) {
  __shared__ float red[4];
  const int m = blockIdx.y;
  const bool valid = m < M_valid;
  const float* tr = t + (size_t)m * K;
  float* xr = x + (size_t)m * K;
  float ss = 0.0f;
  if (valid)
    for (int i = threadIdx.x * 4; i < K; i += 1024) {
      const float4 f = *(const float4*)(tr + i);
      ss += f.x * f.x;
      ss += f.y * f.y;
      ss += f.z * f.z;
      ss += f.w * f.w;
    }
  ss = group_sum(ss, red);
  const float r = rsqrtf(ss / (float)K + eps);
  const int lane16 = threadIdx.x & 15, sub = threadIdx.x >> 4;
  float s2 = 0.0f;
  if (valid)
    for (int sb = sub; sb < K / 256; sb += 16) {
      const int base = sb * 256 + 16 * lane16;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 xo = *(const float4*)(xr + base + 4 * i), to = *(const float4*)(tr + base + 4 * i),
                     wo = *(const float4*)(w + base + 4 * i);
        float4 v;
        v.x = (xo.x + to.x * r * wo.x) * s;
        v.y = (xo.y + to.y * r * wo.y) * s;
        v.z = (xo.z + to.z * r * wo.z) * s;
        v.w = (xo.w + to.w * r * wo.w) * s;
        s2 += v.x * v.x;
        s2 += v.y * v.y;
        s2 += v.z * v.z;
        s2 += v.w * v.w;
        *(float4*)(xr + base + 4 * i) = v;
      }
    }
  s2 = group_sum(s2, red);
  const float r2 = w2_norm ? rsqrtf(s2 / (float)K + eps) : 1.0f;
  for (int sb = sub; sb < K / 256; sb += 16) {
    const int base = sb * 256 + 16 * lane16;
    float v[16];
    if (valid) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 f = *(const float4*)(xr + base + 4 * i);
        v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
        if (w2_norm) {
          const float4 g = *(const float4*)(w2 + base + 4 * i);
          v[4 * i] = f.x * r2 * g.x; v[4 * i + 1] = f.y * r2 * g.y; v[4 * i + 2] = f.z * r2 * g.z; v[4 * i + 3] = f.w * r2 * g.w;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = 0.0f;
    }
    store_row_quant(v, sb, lane16, m, M, K, act32, aq, asc, absum, q2_aq, q2_sc, q2_ab);
  }
}

// act_usum: au[b][m] = sa * S for every 32-block b and token m of a chunk, S the sum of the block's int8 values
// (absum's two halves): the min term's token-side factor, which the prefill GEMM otherwise forms per work-group and
// step, made once per matmul so that it can go into LDS by DMA.  The same expression as in the kernel: the same bits.
// No counterpart in the reference.  grid (ceil(M / 256) * 256, K / 32), local (256, 1).
extern "C" __global__ __launch_bounds__(256) void act_usum(const float* __restrict__ asc, const short* __restrict__ absum,
                                                           int M, float* __restrict__ au) {
  const int m = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
  if (m >= M) return;
  const float sa = asc[(size_t)b * M + m];
  au[(size_t)b * M + m] = sa * (float)((int)absum[(size_t)(2 * b) * M + m] + (int)absum[(size_t)(2 * b + 1) * M + m]);
}

// q4k_wscales: the row side's scale vectors of a Q4_K / Q5_K matrix (the two share the header plane at hdr_off bytes
// into the raw planes) for the prefill GEMM: ws[b][n] = d * sc_b and, N * K / 32 floats further on, v[b][n] =
// -(dmin * mn_b), the expressions of the kernel's own scale preparation (the same bits), written once in front of a
// matmul of many tokens instead of once per 128-token tile and step.  No counterpart in the reference.
// grid (ceil(N / 256) * 256, K / 256), local (256, 1).
extern "C" __global__ __launch_bounds__(256) void q4k_wscales(const uint8_t* __restrict__ raw, size_t hdr_off, int N, int nsb,
                                                              float* __restrict__ wsv) {
  const int n = blockIdx.x * 256 + threadIdx.x, sb = blockIdx.y;
  if (n >= N) return;
  const uint4 h = *(const uint4*)(raw + hdr_off + ((size_t)n * nsb + sb) * 16);
  const float d = f16_bits_to_f32(h.x), dmin = f16_bits_to_f32(h.x >> 16);
  float* ws = wsv + (size_t)sb * 8 * N + n;
  float* v = ws + (size_t)nsb * 8 * N;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int sc0, sc1, mn0, mn1;
    q4k_scales_pair(h.y, h.z, h.w, j, sc0, sc1, mn0, mn1);
    ws[(size_t)(2 * j) * N] = d * (float)sc0;
    ws[(size_t)(2 * j + 1) * N] = d * (float)sc1;
    v[(size_t)(2 * j) * N] = -(dmin * (float)mn0);
    v[(size_t)(2 * j + 1) * N] = -(dmin * (float)mn1);
  }
}

// The same two vectors as operands of the bf16 matrix instruction (the prefill GEMM's min term, its -DAU=3 form):
// x = x1 + x2 + x3 exactly, each piece a bf16 by truncation (split3).  act_usum_bf16: au[b][m] = (u1 | u2 << 16,
// u3 | u3 << 16) of u = sa * S.  q4k_wscales_bf16: ws[b][n] = d * sc as f32, then v[b][n] = (v1 v1, v2 v2, v3 v3, v1 v2)
// of v = -(dmin * mn), 16 bytes an entry.  Grids as act_usum and q4k_wscales.
extern "C" __global__ __launch_bounds__(256) void act_usum_bf16(const float* __restrict__ asc, const short* __restrict__ absum,
                                                                int M, uint2* __restrict__ au) {
  const int m = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
  if (m >= M) return;
  const float sa = asc[(size_t)b * M + m];
  const float u = sa * (float)((int)absum[(size_t)(2 * b) * M + m] + (int)absum[(size_t)(2 * b + 1) * M + m]);
  uint32_t w0, w1;
  split3(u, w0, w1);
  au[(size_t)b * M + m] = make_uint2(w0, w1 | w1 << 16);
}
extern "C" __global__ __launch_bounds__(256) void q4k_wscales_bf16(const uint8_t* __restrict__ raw, size_t hdr_off, int N, int nsb,
                                                                   float* __restrict__ wsv) {
  const int n = blockIdx.x * 256 + threadIdx.x, sb = blockIdx.y;
  if (n >= N) return;
  const uint4 h = *(const uint4*)(raw + hdr_off + ((size_t)n * nsb + sb) * 16);
  const float d = f16_bits_to_f32(h.x), dmin = f16_bits_to_f32(h.x >> 16);
  float* ws = wsv + (size_t)sb * 8 * N + n;
  uint4* v = (uint4*)(wsv + (size_t)nsb * 8 * N) + (size_t)sb * 8 * N + n;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int sc[2], mn[2];
    q4k_scales_pair(h.y, h.z, h.w, j, sc[0], sc[1], mn[0], mn[1]);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      ws[(size_t)(2 * j + q) * N] = d * (float)sc[q];
      uint32_t w0, w1;
      split3(-(dmin * (float)mn[q]), w0, w1);
      const uint32_t v1 = w0 & 0xFFFFu, v2 = w0 >> 16, v3 = w1;
      v[(size_t)(2 * j + q) * N] = make_uint4(v1 | v1 << 16, v2 | v2 << 16, v3 | v3 << 16, w0);
    }
  }
}

// silu(g) = g / (1 + exp(-g)) (reference zero/kernels/ops.cl:33) or the tanh form of gelu.  The exponential and the
// reciprocal are the hardware's (v_exp_f32 on -g log2 e, v_rcp_f32: an ulp or two each) instead of the library's
// sequences of about 25 instructions an element, which were a third of the SwiGLU kernel's time.
__device__ inline float act_gate(float g, int gelu) {
  if (gelu) return 0.5f * g * (1.0f + tanhf(0.7978845608f * (g + 0.044715f * g * g * g)));
  return g * __frcp_rn(1.0f + __expf(-g));
}

// swiglu_quant: y = silu(gate) * up (or the tanh form of gelu(gate) * up) from rows [gate(F) | up(F)], or the row as it
// is when the matmul before has fused the product (`fused`), quantized with K = F (reference zero/kernels/ops.cl:
// 271-315, same arguments; silu(x) = x / (1 + exp(-x)), ops.cl:33).  grid (256 * G, rows), local (256, 1).
extern "C" __global__ __launch_bounds__(256) void swiglu_quant(const float* __restrict__ gu, int F, int M, int M_valid,
                                                               signed char* __restrict__ aq, float* __restrict__ asc,
                                                               short* __restrict__ absum, int act32, int fused,
                                                               int gelu, int q2_aq, int q2_sc, int q2_ab) {
  const int m = blockIdx.y;
  const bool valid = m < M_valid;
  const float* gr = gu + (size_t)m * (fused ? F : 2 * F);
  const int lane16 = threadIdx.x & 15, sub = threadIdx.x >> 4;
  const int nsb = F >> 8, stride = 16 * gridDim.x;
  // (a thread's superblocks two at a time: the loads of both are issued before the first is worked on)
  for (int s0 = blockIdx.x * 16 + sub; s0 < nsb; s0 += 2 * stride) {
    float4 gv[2][4], uv4[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int s = s0 + h * stride;
      const bool in = valid && s < nsb;
      const int base = (in ? s : 0) * 256 + 16 * lane16;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        gv[h][i] = in ? *(const float4*)(gr + base + 4 * i) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        uv4[h][i] = in && !fused ? *(const float4*)(gr + F + base + 4 * i) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int s = s0 + h * stride;
      if (s >= nsb) break;
      float v[16];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[4 * i] = gv[h][i].x; v[4 * i + 1] = gv[h][i].y; v[4 * i + 2] = gv[h][i].z; v[4 * i + 3] = gv[h][i].w;
      }
      if (valid && !fused) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float uv[4] = {uv4[h][i].x, uv4[h][i].y, uv4[h][i].z, uv4[h][i].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[4 * i + j] = act_gate(v[4 * i + j], gelu) * uv[j];
          }
        }
      }
      store_row_quant(v, s, lane16, m, M, F, act32, aq, asc, absum, q2_aq, q2_sc, q2_ab);
    }
  }
}

// q4k_wscales_int: the row side for chunks with per-256 activation scales (the prefill GEMM's -DAU=4 form): the 6-bit
// sub-block scales as int32 [K / 32][N], the min term's bf16 pieces as q4k_wscales_bf16 writes them, and behind those
// (20 bytes per block and row in) d as f32 [K / 256][N].  Grid as q4k_wscales.
extern "C" __global__ __launch_bounds__(256) void q4k_wscales_int(const uint8_t* __restrict__ raw, size_t hdr_off, int N, int nsb,
                                                                  float* __restrict__ wsv) {
  const int n = blockIdx.x * 256 + threadIdx.x, sb = blockIdx.y;
  if (n >= N) return;
  const uint4 h = *(const uint4*)(raw + hdr_off + ((size_t)n * nsb + sb) * 16);
  const float d = f16_bits_to_f32(h.x), dmin = f16_bits_to_f32(h.x >> 16);
  int* ws = (int*)wsv + (size_t)sb * 8 * N + n;
  uint4* v = (uint4*)(wsv + (size_t)nsb * 8 * N) + (size_t)sb * 8 * N + n;
  wsv[(size_t)nsb * 8 * N * 5 + (size_t)sb * N + n] = d;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int sc[2], mn[2];
    q4k_scales_pair(h.y, h.z, h.w, j, sc[0], sc[1], mn[0], mn[1]);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      ws[(size_t)(2 * j + q) * N] = sc[q];
      uint32_t w0, w1;
      split3(-(dmin * (float)mn[q]), w0, w1);
      const uint32_t v1 = w0 & 0xFFFFu, v2 = w0 >> 16, v3 = w1;
      v[(size_t)(2 * j + q) * N] = make_uint4(v1 | v1 << 16, v2 | v2 << 16, v3 | v3 << 16, w0);
    }
  }
}

// ---- the fused producers over chunks of many rows: a work-group takes 16 consecutive rows one after the other and
// keeps their scales and sums in LDS, [block][16 rows], so that the token-minor arrays are written in pieces of 16
// rows (64 and 32 bytes) instead of one element per block and row from a work-group per row, whose 480 scattered
// stores a row were most of that form's memory transactions.  One-pass engines, M a multiple of 16, rows of up to
// R16_KMAX (R16_KMAX_NORM) values.
#define R16_KMAX 20480      // swiglu_quant_r16 (80 KiB of LDS: two work-groups a compute unit)
#define R16_KMAX_NORM 16384 // rmsnorm_quant_r16 (64 KiB, and the row sum's four floats)
template <int KMAX> struct R16Stage {
  float sc[KMAX / 32 * 16];
  short sum[KMAX / 16 * 16];
};
// a thread's 16 values of superblock s of row r of the 16: quantized, the int8 values stored, scale and sum staged
template <int KMAX>
__device__ inline void r16_quant(R16Stage<KMAX>& st, const float* v, int s, int lane16, int r, int m, int K, int act32,
                                 signed char* __restrict__ aq) {
  const float amax = block_amax(v, act32);
  uint4 pk;
  int sum;
  quant16(v, amax, pk, sum, nullptr);
  *(uint4*)(aq + (size_t)m * K + s * 256 + 16 * lane16) = pk;
  st.sum[(s * 16 + lane16) * 16 + r] = (short)sum;
  if (act32) {
    if ((lane16 & 1) == 0) st.sc[(s * 8 + (lane16 >> 1)) * 16 + r] = amax / 127.0f;
  } else if (lane16 == 0) {
    st.sc[s * 16 + r] = amax / 127.0f;
  }
}
// the staged scales and sums of rows m0 .. m0 + 15 out to asc [blocks][M] and absum [K / 16][M]
template <int KMAX>
__device__ inline void r16_flush(const R16Stage<KMAX>& st, int m0, int M, int K, int act32, float* __restrict__ asc,
                                 short* __restrict__ absum) {
  __syncthreads();
  const int nb = act32 ? K >> 5 : K >> 8;
  for (int i = threadIdx.x; i < nb * 16; i += 256) asc[(size_t)(i >> 4) * M + m0 + (i & 15)] = st.sc[i];
  for (int i = threadIdx.x; i < (K >> 4) * 8; i += 256)
    *(uint32_t*)(absum + (size_t)(i >> 3) * M + m0 + 2 * (i & 7)) = *(const uint32_t*)(st.sum + (i >> 3) * 16 + 2 * (i & 7));
}

// rmsnorm_quant over 16 rows a work-group: grid (256, M / 16).  A row stays in registers between its sum of squares
// and its quantization, and the next row's loads are in flight meanwhile.
extern "C" __global__ __launch_bounds__(256, 2) void rmsnorm_quant_r16(const float* __restrict__ x, int row_off,
                                                                       const float* __restrict__ w, int K, int M,
                                                                       int M_valid, float eps, signed char* __restrict__ aq,
                                                                       float* __restrict__ asc, short* __restrict__ absum,
                                                                       float* __restrict__ hout, int write_h, int act32) {
  __shared__ float red[4];
  __shared__ R16Stage<R16_KMAX_NORM> st;
  const int m0 = blockIdx.y * 16;
  const int lane16 = threadIdx.x & 15, sub = threadIdx.x >> 4, nsb = K >> 8;
  constexpr int MAXU = R16_KMAX_NORM / 4096;  // superblocks a thread holds
  auto load = [&](float4 (&xv)[MAXU][4], int m) {
    const bool valid = m < M_valid;
    const float* xr = x + (size_t)((valid ? m : 0) + row_off) * K;
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      const int sb = sub + 16 * u;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        xv[u][i] = valid && sb < nsb ? *(const float4*)(xr + sb * 256 + 16 * lane16 + 4 * i) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  };
  auto work = [&](const float4 (&xv)[MAXU][4], int r) {
    const int m = m0 + r;
    float ss = 0.0f;
#pragma unroll
    for (int u = 0; u < MAXU; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ss += xv[u][i].x * xv[u][i].x;
        ss += xv[u][i].y * xv[u][i].y;
        ss += xv[u][i].z * xv[u][i].z;
        ss += xv[u][i].w * xv[u][i].w;
      }
    ss = group_sum(ss, red);
    const float rs = rsqrtf(ss / (float)K + eps);
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      const int sb = sub + 16 * u;
      if (sb >= nsb) break;  // (the same for the 16 threads of a superblock)
      const int base = sb * 256 + 16 * lane16;
      float v[16];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 f = xv[u][i], g = *(const float4*)(w + base + 4 * i);
        v[4 * i] = f.x * rs * g.x; v[4 * i + 1] = f.y * rs * g.y; v[4 * i + 2] = f.z * rs * g.z; v[4 * i + 3] = f.w * rs * g.w;
      }
      if (write_h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          *(float4*)(hout + (size_t)m * K + base + 4 * i) = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
      r16_quant(st, v, sb, lane16, r, m, K, act32, aq);
    }
  };
  float4 xa[MAXU][4], xb[MAXU][4];
  load(xa, m0);
#pragma unroll 1
  for (int r = 0; r < 16; r += 2) {
    load(xb, m0 + r + 1);
    work(xa, r);
    load(xa, min(m0 + r + 2, m0 + 15));  // (after the last pair: row 15 again, not used)
    work(xb, r + 1);
  }
  r16_flush(st, m0, M, K, act32, asc, absum);
}

// swiglu_quant over 16 rows a work-group: grid (256, M / 16).
extern "C" __global__ __launch_bounds__(256, 2) void swiglu_quant_r16(const float* __restrict__ gu, int F, int M, int M_valid,
                                                                      signed char* __restrict__ aq, float* __restrict__ asc,
                                                                      short* __restrict__ absum, int act32, int fused,
                                                                      int gelu) {
  __shared__ R16Stage<R16_KMAX> st;
  const int m0 = blockIdx.y * 16;
  const int lane16 = threadIdx.x & 15, sub = threadIdx.x >> 4, nsb = F >> 8;
  // (the units of work: superblock s of row r, row-major over the 16 rows, dealt to the 16 groups of threads in turn --
  //  by rows alone 20 superblocks would keep four groups busy twice and twelve once; the loads of a thread's next unit
  //  are in flight while it works on the current one)
  const int units = 16 * nsb, total = (units - sub + 15) / 16;
  struct Unit { float4 g[4], u[4]; int r, s; };
  auto load = [&](Unit& t, int j) {
    const int i = sub + 16 * min(j, total - 1);   // (past the end: the last again, not used)
    t.r = i / nsb;
    t.s = i - t.r * nsb;
    const bool in = m0 + t.r < M_valid;
    const float* gr = gu + (size_t)(in ? m0 + t.r : 0) * (fused ? F : 2 * F) + t.s * 256 + 16 * lane16;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      t.g[k] = in ? *(const float4*)(gr + 4 * k) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      t.u[k] = in && !fused ? *(const float4*)(gr + F + 4 * k) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  };
  auto work = [&](const Unit& t) {
    float v[16];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[4 * k] = t.g[k].x; v[4 * k + 1] = t.g[k].y; v[4 * k + 2] = t.g[k].z; v[4 * k + 3] = t.g[k].w;
    }
    if (m0 + t.r < M_valid && !fused) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float uv[4] = {t.u[k].x, t.u[k].y, t.u[k].z, t.u[k].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) v[4 * k + j] = act_gate(v[4 * k + j], gelu) * uv[j];
      }
    }
    r16_quant(st, v, t.s, lane16, t.r, m0 + t.r, F, act32, aq);
  };
  if (total > 0) {
    Unit a, b;
    load(a, 0);
#pragma unroll 1
    for (int j = 0; j < total; j += 2) {
      load(b, j + 1);
      work(a);
      load(a, j + 2);
      if (j + 1 < total) work(b);
    }
  }
  r16_flush(st, m0, M, F, act32, asc, absum);
}

// softcap_rows: C[t][off + n] = cap * tanh(C[t][off + n] / cap) over N columns of the launch's rows (the output head of
// a two-pass engine: the cap applies to the sum of both passes; reference zero/engine.h:1103-1110).
// grid (ceil(N / 256) * 256, T).
extern "C" __global__ void softcap_rows(float* C, int ld, int off, int N, float cap) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
  if (n >= N) return;
  float* p = C + (size_t)t * ld + off + n;
  *p = head_out(*p, cap);
}

// asc_expand: per-256 activation scales a256 [nsb][M] written out per 32-block, a32 [nsb * 8][M] (each scale eight
// times): the matmul kernels take per-32 scales, and a chunk quantized with one scale per superblock (the reference's
// act32 = 0, zero/kernels/ops.cl:38-72 and the non-ACT32 GEMM, zero/kernels/gemm.cl:489-520) runs through them with the
// same integer sums and the same scale on each of a superblock's blocks.  grid: ceil(nsb * 8 * M / 256) x 256.
extern "C" __global__ void asc_expand(const float* __restrict__ a256, float* __restrict__ a32, int M, int nsb) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)nsb * 8 * M) return;
  const size_t row = i / M, m = i - row * M;
  a32[i] = a256[(row >> 3) * M + m];
}

// fill32: p[i] = v for i < n (the fill used where a captured graph must not hold a memset node).
extern "C" __global__ void fill32(uint32_t* p, uint32_t v, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// copy128: dst[i] = src[i] over n 16-byte units; the plain streaming copy the bandwidth probe and the counter
// calibration use.
extern "C" __global__ void copy128(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

// read_probe: streams n 16-byte units and folds them into one word per thread (written only if it is the impossible
// value, so the loads cannot be dropped): the read-bandwidth probe (the reference's Engine::read_gbs pattern,
// zero/engine.h:154-208).
extern "C" __global__ void read_probe(const uint4* __restrict__ src, size_t n, uint32_t* sink) {
  uint32_t acc = 0;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const uint4 v = src[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9E3779B9u) sink[0] = acc;
}

// mfma_probe: register-resident int8 matrix instructions, four independent 32x32x32 accumulators per wave, `iters`
// rounds: the issue-rate ceiling of the int8 matrix pipe that the GEMM figures are set against (the reference measures
// its own in bench/gpu_bench.cpp:10-15).  2 * 32*32*32 * 4 * iters operations per wave.
extern "C" __global__ __launch_bounds__(256) void mfma_probe(uint32_t* sink, int iters) {
  v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, (int)blockIdx.x, 7};
  v16i c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int i = 0; i < iters; ++i) {
    c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, a, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, b, c3, 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) s ^= c0[i] ^ c1[i] ^ c2[i] ^ c3[i];
  if (s == 0x12345678) sink[0] = (uint32_t)s;
}
