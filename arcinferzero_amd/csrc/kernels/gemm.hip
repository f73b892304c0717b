// "gemm" module: the prefill GEMM  C[m][c_off + n] (=, +=, silu(C) *) sum_k A[m][k] W[n][k]  on int8 MFMA, for dense
// matrices and for the expert-grouped tiles of a mixture-of-experts layer.
//
// Arithmetic (reference zero/kernels/gemm.cl:439-488, the per-32 activation scale form): every 32-block b of K gives
// an exact int32 sum I[m][n][b] (v_mfma_i32_32x32x32_i8, accumulator cleared per block; Q6_K: two K = 16 products per
// block, one per 16-element sub-scale), then in f32
//   Q8_0 : res += (sa[m][b] * d[n][b]) * (float)I
//   Q4_K : res += (sa[m][b] * (d[n] * sc[n][b])) * (float)I  -  (sa[m][b] * (float)S[m][b]) * (dmin[n] * mn[n][b])
//   Q6_K : res += (sa[m][b] * (d[n] * sc16[n][h])) * (float)I_h      for both halves h of the block
// with S the sum of the block's 32 int8 activations (absum pairs).  Blocks are added in K order.
//
// Tiling: a work-group of 256 threads (4 waves, 2 x 2) computes 128 tokens x 128 weight rows; each wave 64 x 64 as
// 2 x 2 MFMA tiles.  K advances in half superblocks (128 values): the tokens' int8 values and the weight rows,
// decoded to int8 once per work-group, are staged in LDS with a 16-byte row pad (conflict-free 128-bit reads), next
// to the activation scales and the weight scales as f32.  The MFMA's A operand is the token tile and B the weight
// tile, so a lane owns one weight row n and writes 128-byte runs of C.
#include "common.h"

#define BM 128
#define BN 128
#define BK 128
#define LDS_PAD 16

template <int QT> struct GemmLds {
  uint8_t act[BM][BK + LDS_PAD];
  uint8_t wq[BN][BK + LDS_PAD];
  float sa[4][BM];
  float u[4][BM];
  float wsc[8][BN];  // per 16-element half block (Q4_K / Q8_0: the block's scale twice)
  float wmn[4][BN];
  int ssum[4][BM];  // Q4_K: sum of each block's 32 int8 activations
  int rowmap[BM];
};

// Decodes the half superblock (s, hh) of BN weight rows starting at row n0 (of `rows_total` plane rows) into LDS.
template <int QT>
__device__ inline void stage_weights(GemmLds<QT>& L, const uint8_t* __restrict__ raw, size_t rows_total, int nsb,
                                     size_t row_base, int n0, int N, int s, int hh) {
  const int t = threadIdx.x;
  if constexpr (QT == QT_Q4_K) {
    const PlanesQ4K pl = planes_q4k(rows_total, nsb);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const int n = min(n0 + row, N - 1);
      const int j = 2 * hh + (c >> 1), half = c & 1;
      const uint4 w = *(const uint4*)(raw + pl.qs + ((row_base + n) * nsb + s) * 128 + 32 * j + 16 * half);
      const int off = 64 * (c >> 1) + 16 * half;
      *(uint4*)&L.wq[row][off] = make_uint4(w.x & 0x0F0F0F0Fu, w.y & 0x0F0F0F0Fu, w.z & 0x0F0F0F0Fu, w.w & 0x0F0F0F0Fu);
      *(uint4*)&L.wq[row][off + 32] = make_uint4((w.x >> 4) & 0x0F0F0F0Fu, (w.y >> 4) & 0x0F0F0F0Fu,
                                                 (w.z >> 4) & 0x0F0F0F0Fu, (w.w >> 4) & 0x0F0F0F0Fu);
    }
    {
      const int row = t >> 1, p = t & 1;
      const int n = min(n0 + row, N - 1);
      const uint4 h = *(const uint4*)(raw + pl.hdr + ((row_base + n) * nsb + s) * 16);
      const float d = f16_bits_to_f32(h.x), dmin = f16_bits_to_f32(h.x >> 16);
      int sc0, sc1, mn0, mn1;
      q4k_scales_pair(h.y, h.z, h.w, 2 * hh + p, sc0, sc1, mn0, mn1);
      L.wsc[4 * p + 0][row] = L.wsc[4 * p + 1][row] = d * (float)sc0;
      L.wsc[4 * p + 2][row] = L.wsc[4 * p + 3][row] = d * (float)sc1;
      L.wmn[2 * p][row] = dmin * (float)mn0;
      L.wmn[2 * p + 1][row] = dmin * (float)mn1;
    }
  } else if constexpr (QT == QT_Q6_K) {
    const PlanesQ6K pl = planes_q6k(rows_total, nsb);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const int n = min(n0 + row, N - 1);
      const size_t rs = (row_base + n) * nsb + s;
      const int l0 = 16 * c, q1 = l0 >> 5;
      const uint4 Lq = *(const uint4*)(raw + pl.ql + rs * 128 + 64 * hh + l0);
      const uint4 Hq = *(const uint4*)(raw + pl.qh + rs * 64 + 32 * hh + (l0 & 31));
      const uint32_t Lw[4] = {Lq.x, Lq.y, Lq.z, Lq.w}, Hw[4] = {Hq.x, Hq.y, Hq.z, Hq.w};
      uint32_t w1[4], w2[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        w1[k] = sub32_bytes((Lw[k] & 0x0F0F0F0Fu) | (((Hw[k] >> (2 * q1)) & 0x03030303u) << 4));
        w2[k] = sub32_bytes(((Lw[k] >> 4) & 0x0F0F0F0Fu) | (((Hw[k] >> (2 * q1 + 4)) & 0x03030303u) << 4));
      }
      *(uint4*)&L.wq[row][l0] = make_uint4(w1[0], w1[1], w1[2], w1[3]);
      *(uint4*)&L.wq[row][64 + l0] = make_uint4(w2[0], w2[1], w2[2], w2[3]);
    }
    {
      const int row = t >> 1, p = t & 1;
      const int n = min(n0 + row, N - 1);
      const size_t rs = (row_base + n) * nsb + s;
      const float d = f16_bits_to_f32(*(const unsigned short*)(raw + pl.d + rs * 2));
      const uint32_t sc4 = *(const uint32_t*)(raw + pl.sc + rs * 16 + 8 * hh + 4 * p);
#pragma unroll
      for (int k = 0; k < 4; ++k) L.wsc[4 * p + k][row] = d * (float)(int)(signed char)((sc4 >> (8 * k)) & 0xFF);
    }
  } else {
    const PlanesQ80 pl = planes_q80(rows_total, nsb);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id = t + 256 * i, row = id >> 3, c = id & 7;
      const int n = min(n0 + row, N - 1);
      *(uint4*)&L.wq[row][16 * c] = *(const uint4*)(raw + pl.qs + ((row_base + n) * nsb + s) * 256 + 128 * hh + 16 * c);
    }
    {
      const int row = t >> 1, p = t & 1;
      const int n = min(n0 + row, N - 1);
      const uint32_t d2 = *(const uint32_t*)(raw + pl.d + (((row_base + n) * nsb + s) * 8 + 4 * hh + 2 * p) * 2);
      L.wsc[4 * p + 0][row] = L.wsc[4 * p + 1][row] = f16_bits_to_f32(d2);
      L.wsc[4 * p + 2][row] = L.wsc[4 * p + 3][row] = f16_bits_to_f32(d2 >> 16);
    }
  }
}

// Stages the tokens' int8 values, scales and (Q4_K) scaled sums of the half superblock.  Row r of the tile is token
// row L.rowmap[r] (or -1: a row past the tile, staged as zeros).  The block sums of the activations that the Q4_K min
// term needs are taken from the int8 values as they pass (the same integers the quantizer's absum holds), so the
// expert inputs, which come without sums, take the same path.
template <int QT>
__device__ inline void stage_acts(GemmLds<QT>& L, const signed char* __restrict__ aq, const float* __restrict__ asc,
                                  int M, int K, int s, int hh) {
  const int t = threadIdx.x;
  const int e0 = s * 256 + 128 * hh;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int id = t + 256 * i, row = id >> 3, c = id & 7;
    const int m = L.rowmap[row];
    uint4 v = make_uint4(0, 0, 0, 0);
    if (m >= 0) v = *(const uint4*)(aq + (size_t)m * K + e0 + 16 * c);
    *(uint4*)&L.act[row][16 * c] = v;
    if constexpr (QT == QT_Q4_K) {
      int sh = dot4(v.x, 0x01010101u, 0);
      sh = dot4(v.y, 0x01010101u, sh);
      sh = dot4(v.z, 0x01010101u, sh);
      sh = dot4(v.w, 0x01010101u, sh);
      const int S = sh + __shfl_xor(sh, 1, 64);
      if ((c & 1) == 0) L.ssum[c >> 1][row] = S;
    }
  }
  if constexpr (QT == QT_Q4_K) __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int id = t + 256 * i, b = id >> 7, row = id & 127;
    const int m = L.rowmap[row];
    const int gb = s * 8 + 4 * hh + b;
    const float sa = m >= 0 ? asc[(size_t)gb * M + m] : 0.0f;
    L.sa[b][row] = sa;
    if constexpr (QT == QT_Q4_K) L.u[b][row] = sa * (float)L.ssum[b][row];
  }
}

template <int QT, bool TILES>
__device__ inline void gemm_body(const uint8_t* __restrict__ raw, const signed char* __restrict__ aq,
                                 const float* __restrict__ asc, const short* __restrict__ absum, float* __restrict__ C,
                                 int M, int N, int K, int ldc, int c_off, int accumulate, int s_begin, int s_end,
                                 size_t rows_total, size_t row_base, int m0, int rows_valid, int n0,
                                 const int* __restrict__ rowmap, int use_map, const float* __restrict__ rowscale,
                                 int use_scale) {
  __shared__ GemmLds<QT> L;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  if (t < BM) {
    int m = -1;
    if (t < rows_valid) m = (TILES && use_map) ? rowmap[m0 + t] : m0 + t;
    L.rowmap[t] = m;
  }
  __syncthreads();

  v16f res[2][2];
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int ns = 0; ns < 2; ++ns)
#pragma unroll
      for (int i = 0; i < 16; ++i) res[ms][ns][i] = 0.0f;

  for (int s = s_begin; s < s_end; ++s) {
#pragma unroll 1
    for (int hh = 0; hh < 2; ++hh) {
      stage_weights<QT>(L, raw, rows_total, nsb, row_base, n0, N, s, hh);
      stage_acts<QT>(L, aq, asc, M, K, s, hh);
      __syncthreads();
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        float wscale[2][2], wmin[2];
#pragma unroll
        for (int ns = 0; ns < 2; ++ns) {
          const int nl = wn * 64 + ns * 32 + l32;
          wscale[ns][0] = L.wsc[2 * b][nl];
          wscale[ns][1] = L.wsc[2 * b + 1][nl];
          wmin[ns] = QT == QT_Q4_K ? L.wmn[b][nl] : 0.0f;
        }
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
          const int mrow = wm * 64 + ms * 32;
          // the 16 token rows this lane's accumulators belong to: 8 * (i / 4) + 4 * g + i % 4
          float sav[16], uv[16];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float4 s4 = *(const float4*)&L.sa[b][mrow + 8 * q + 4 * g];
            sav[4 * q] = s4.x; sav[4 * q + 1] = s4.y; sav[4 * q + 2] = s4.z; sav[4 * q + 3] = s4.w;
            if constexpr (QT == QT_Q4_K) {
              const float4 u4 = *(const float4*)&L.u[b][mrow + 8 * q + 4 * g];
              uv[4 * q] = u4.x; uv[4 * q + 1] = u4.y; uv[4 * q + 2] = u4.z; uv[4 * q + 3] = u4.w;
            }
          }
#pragma unroll
          for (int ns = 0; ns < 2; ++ns) {
            const int nl = wn * 64 + ns * 32 + l32;
            if constexpr (QT == QT_Q6_K) {
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                const long a8 = *(const long*)&L.act[mrow + l32][32 * b + 16 * h + 8 * g];
                const long w8 = *(const long*)&L.wq[nl][32 * b + 16 * h + 8 * g];
                v16i z;
#pragma unroll
                for (int i = 0; i < 16; ++i) z[i] = 0;
                const v16i I = __builtin_amdgcn_mfma_i32_32x32x16_i8(a8, w8, z, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 16; ++i) res[ms][ns][i] += (sav[i] * wscale[ns][h]) * (float)I[i];
              }
            } else {
              const v4i a16 = *(const v4i*)&L.act[mrow + l32][32 * b + 16 * g];
              const v4i w16 = *(const v4i*)&L.wq[nl][32 * b + 16 * g];
              v16i z;
#pragma unroll
              for (int i = 0; i < 16; ++i) z[i] = 0;
              const v16i I = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16, w16, z, 0, 0, 0);
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                res[ms][ns][i] += (sav[i] * wscale[ns][0]) * (float)I[i];
                if constexpr (QT == QT_Q4_K) res[ms][ns][i] -= uv[i] * wmin[ns];
              }
            }
          }
        }
      }
      __syncthreads();
    }
  }

  // ---- epilogue: lane = weight row n, accumulator i = token row 8 * (i / 4) + 4 * g + i % 4
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int ns = 0; ns < 2; ++ns) {
      const int n = n0 + wn * 64 + ns * 32 + l32;
      if (n >= N) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = wm * 64 + ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
        if (r >= rows_valid) continue;
        float v = res[ms][ns][i];
        if (TILES && use_scale) v *= rowscale[m0 + r];
        float* cp = C + (size_t)(m0 + r) * ldc + c_off + n;
        if (accumulate == 1) {
          v += *cp;
        } else if (accumulate == 2) {  // fused SwiGLU: C holds the gate projection, v the up projection
          const float gt = *cp;
          v *= gt / (1.0f + __expf(-gt));
        }
        *cp = v;
      }
    }
}

// gemm, dense.  Arguments as the reference's (zero/kernels/gemm.cl:163-166); with the weights decoded in the kernel
// its (wq, wh) pair is (raw planes, unused), and rgroup (its cache-blocking knob) is accepted and ignored.
// grid: (ceil(N / 128) * ceil(M / 128)) work-groups of 256 threads, token tiles fastest.
#define GEMM_INST(QT)                                                                                                \
  extern "C" __global__ __launch_bounds__(256) void gemm__QTYPE##QT##_ACT321(                                         \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {        \
    const int mt = (M + BM - 1) / BM;                                                                                 \
    const int tm = blockIdx.x % mt, tn = blockIdx.x / mt;                                                             \
    const int m0 = tm * BM, n0 = tn * BN;                                                                             \
    gemm_body<QT, false>(raw, aq, asc, absum, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,   \
                         min(BM, M - m0), n0, nullptr, 0, nullptr, 0);                                                \
  }

// gemm over expert tiles (reference zero/kernels/gemm.cl:146-161, -DMOE_TILES): W holds all experts' rows (N each);
// tile t of the list = (expert, first slot, rows <= 128) from moe_scan; slot r reads token row rowmap[r] (use_map) or
// r, writes C row r, times rowscale[r] (use_scale).  Experts [e0, e1).  grid (ceil(N / 128), tile work-groups):
// work-group y loops over tiles y, y + gridDim.y, ...
#define GEMM_TILES_INST(QT)                                                                                          \
  extern "C" __global__ __launch_bounds__(256) void gemm__QTYPE##QT##_ACT321_MOE_TILES1(                              \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int accumulate, const int* tiles, const int* tstart, int e0, int e1,    \
      const int* rowmap, int use_map, const float* rowscale, int use_scale, int NE) {                                 \
    const int t_end = tstart[e1];                                                                                     \
    for (int ti = tstart[e0] + blockIdx.y; ti < t_end; ti += gridDim.y) {                                             \
      const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];                                \
      gemm_body<QT, true>(raw, aq, asc, absum, C, M, N, K, ldc, 0, accumulate, 0, K >> 8, (size_t)NE * N,             \
                          (size_t)e * N, r0, min(nr, BM), blockIdx.x * BN, rowmap, use_map, rowscale, use_scale);     \
      __syncthreads();                                                                                                \
    }                                                                                                                 \
  }

GEMM_INST(8)
GEMM_INST(12)
GEMM_INST(14)
GEMM_TILES_INST(8)
GEMM_TILES_INST(12)
GEMM_TILES_INST(14)
