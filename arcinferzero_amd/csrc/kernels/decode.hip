// "decode" module: the bandwidth-bound matrix-vector products on the raw weight planes, for 1 token (gemv) and for
// 2..8 tokens that share one read of the weights (gemv_mt).
//
// Arithmetic per 16-element half block h of weight row n and token t, as the reference's gemv
// (zero/kernels/decode.cl:992-1003):  I = sum of 16 int8 x int8 products (v_dot4_i32_i8, exact int32);
//   Q4_K : acc += sa * (d * (float)(sc * I) - dmin * (float)(mn * bs))      sa: the token's scale of the 32-block,
//   Q5_K : as Q4_K, the values 0..31 (the fifth bits come from their own plane)
//   Q6_K : acc += sa * d * (float)(sc16 * I)                                bs: its int16 sum of the 16 activations
//   Q8_0 : acc += sa * d * (float)I
//   IQ4_XS: acc += sa * d * (float)(ls * I)      ls: the block's 6-bit scale - 32; values through the 16-entry table
// (the reference groups the two halves of a 32-block inside the int -> float conversion; here each half is converted
// alone, because a lane's 16-byte unit of Q4_K nibbles holds halves of two different blocks: the same real number,
// rounded at another place).  Lanes add their terms in unit order; a row's 32 lanes are summed by a fixed tree.
//
// Mapping: a half wave (32 lanes) takes GROWS consecutive rows; lane l reads the 16-byte units l, l+32, ... of a
// row's quant plane, so a wave's load instruction covers two contiguous 512-byte runs.  The token's int8 values,
// scales and sums of a unit are loaded once and used for all GROWS rows.
#include "common.h"
#include "route1.h"

template <int QT> struct UnitsPerSb { static constexpr int v = QT == QT_Q8_0 ? 16 : 8; };

// IQ3_S: the codebook (512 entries of four magnitudes 1, 3, ..., 15, one per byte; ggml's iq3s_grid) in LDS, copied from
// the kernels' `tabs` argument once per work-group, before anything else (every thread of the work-group calls this).
// IQ3_XXS: its 256 entries (magnitudes 4, 12, ..., 52, 62; ggml's iq3xxs_grid) lie behind those in `tabs` and take the
// array's first 256 words.
__shared__ uint32_t iq3s_grid_lds[512];
__device__ inline void iq3s_grid_init(const uint32_t* __restrict__ tabs) {
  for (int i = threadIdx.x; i < 512; i += blockDim.x) iq3s_grid_lds[i] = tabs[i];
  __syncthreads();
}
template <int QT>
__device__ inline void grid_init(const uint32_t* __restrict__ tabs) {
  if constexpr (QT == QT_IQ3_S) iq3s_grid_init(tabs);
  if constexpr (QT == QT_IQ3_XXS) {
    for (int i = threadIdx.x; i < 256; i += blockDim.x) iq3s_grid_lds[i] = tabs[512 + i];
    __syncthreads();
  }
}

// acc[r][t] += the products of plane rows rows[r] (absolute rows of planes that hold `plane_rows` rows) with the token
// rows tok[t] of aq / asc / absum, this half wave's share (lane hl takes the 16-byte units hl, hl + 32, ...).
// SPLIT < GROWS: rows[SPLIT..GROWS) are rows of a second set of planes of the same shape, raw2 (the gate and the up
// experts in one pass: the token's values are loaded once for both, and both matrices' loads are in flight together).
template <int QT, int TB, int GROWS, int SPLIT = GROWS>
__device__ __forceinline__ void gemv_acc(const uint8_t* __restrict__ raw, size_t plane_rows, const size_t (&rows)[GROWS], int K,
                                         const int (&tok)[TB], const signed char* __restrict__ aq,
                                         const float* __restrict__ asc, const short* __restrict__ absum, int M, int hl,
                                         float (&acc)[GROWS][TB], int nt = TB, const uint8_t* __restrict__ raw2 = nullptr) {
  const int nsb = K >> 8, units = nsb * UnitsPerSb<QT>::v;
  if constexpr (QT == QT_Q4_K || QT == QT_Q5_K) {
    const PlanesQ4K pl = planes_q4k(plane_rows, nsb);
    const int j = (hl >> 1) & 3, half = hl & 1;
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 3;
      const int e_lo = sb * 256 + 64 * j + 16 * half;
      uint4 alo[TB], ahi[TB];
      float salo[TB], sahi[TB];
      int bslo[TB], bshi[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        alo[t] = *(const uint4*)(aq + (size_t)tt * K + e_lo);
        ahi[t] = *(const uint4*)(aq + (size_t)tt * K + e_lo + 32);
        salo[t] = asc[(size_t)(sb * 8 + 2 * j) * M + tt];
        sahi[t] = asc[(size_t)(sb * 8 + 2 * j + 1) * M + tt];
        bslo[t] = absum[(size_t)(sb * 16 + 4 * j + half) * M + tt];
        bshi[t] = absum[(size_t)(sb * 16 + 4 * j + 2 + half) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const uint4 w = *(const uint4*)(rb + pl.qs + n * nsb * 128 + (size_t)u * 16);
        const uint4 h = *(const uint4*)(rb + pl.hdr + (n * nsb + sb) * 16);
        const float d = f16_bits_to_f32(h.x), dmin = f16_bits_to_f32(h.x >> 16);
        int sc0, sc1, mn0, mn1;
        q4k_scales_pair(h.y, h.z, h.w, j, sc0, sc1, mn0, mn1);
        uint32_t wl[4] = {w.x & 0x0F0F0F0Fu, w.y & 0x0F0F0F0Fu, w.z & 0x0F0F0F0Fu, w.w & 0x0F0F0F0Fu};
        uint32_t wh[4] = {(w.x >> 4) & 0x0F0F0F0Fu, (w.y >> 4) & 0x0F0F0F0Fu, (w.z >> 4) & 0x0F0F0F0Fu,
                          (w.w >> 4) & 0x0F0F0F0Fu};
        if constexpr (QT == QT_Q5_K) {  // the fifth bits of the unit's 32 values
          const uint32_t H = *(const uint32_t*)(rb + pl.qh + n * nsb * 32 + (size_t)u * 4), ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
          for (int k = 0; k < 4; ++k) { wl[k] = q5k_lo(ww[k], H, k); wh[k] = q5k_hi(ww[k], H, k); }
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int ilo = dot4(wl[0], alo[t].x, 0);
          ilo = dot4(wl[1], alo[t].y, ilo);
          ilo = dot4(wl[2], alo[t].z, ilo);
          ilo = dot4(wl[3], alo[t].w, ilo);
          int ihi = dot4(wh[0], ahi[t].x, 0);
          ihi = dot4(wh[1], ahi[t].y, ihi);
          ihi = dot4(wh[2], ahi[t].z, ihi);
          ihi = dot4(wh[3], ahi[t].w, ihi);
          acc[r][t] += salo[t] * (d * (float)(sc0 * ilo) - dmin * (float)(mn0 * bslo[t]));
          acc[r][t] += sahi[t] * (d * (float)(sc1 * ihi) - dmin * (float)(mn1 * bshi[t]));
        }
      }
    }
  } else if constexpr (QT == QT_Q6_K) {
    const PlanesQ6K pl = planes_q6k(plane_rows, nsb);
    const int idx = hl & 7, n2 = idx >> 2, l0 = (idx & 3) * 16, q1 = l0 >> 5;
    const int hsh1 = 2 * q1, hsh2 = 2 * q1 + 4;
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 3;
      const int e1 = sb * 256 + 128 * n2 + l0, e2 = e1 + 64;
      uint4 a1[TB], a2[TB];
      float sa1[TB], sa2[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        a1[t] = *(const uint4*)(aq + (size_t)tt * K + e1);
        a2[t] = *(const uint4*)(aq + (size_t)tt * K + e2);
        sa1[t] = asc[(size_t)(e1 >> 5) * M + tt];
        sa2[t] = asc[(size_t)(e2 >> 5) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const size_t rs = n * nsb + sb;
        const uint4 L = *(const uint4*)(rb + pl.ql + n * nsb * 128 + (size_t)u * 16);
        const uint4 H = *(const uint4*)(rb + pl.qh + rs * 64 + 32 * n2 + (l0 & 31));
        const signed char* scp = (const signed char*)(rb + pl.sc + rs * 16 + 8 * n2 + (idx & 3));
        const int sc1 = scp[0], sc2 = scp[4];
        const float d = f16_bits_to_f32(*(const unsigned short*)(rb + pl.d + rs * 2));
        const uint32_t Lw[4] = {L.x, L.y, L.z, L.w}, Hw[4] = {H.x, H.y, H.z, H.w};
        uint32_t w1[4], w2[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          w1[k] = sub32_bytes((Lw[k] & 0x0F0F0F0Fu) | (((Hw[k] >> hsh1) & 0x03030303u) << 4));
          w2[k] = sub32_bytes(((Lw[k] >> 4) & 0x0F0F0F0Fu) | (((Hw[k] >> hsh2) & 0x03030303u) << 4));
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int i1 = dot4(w1[0], a1[t].x, 0);
          i1 = dot4(w1[1], a1[t].y, i1);
          i1 = dot4(w1[2], a1[t].z, i1);
          i1 = dot4(w1[3], a1[t].w, i1);
          int i2 = dot4(w2[0], a2[t].x, 0);
          i2 = dot4(w2[1], a2[t].y, i2);
          i2 = dot4(w2[2], a2[t].z, i2);
          i2 = dot4(w2[3], a2[t].w, i2);
          acc[r][t] += sa1[t] * d * (float)(sc1 * i1);
          acc[r][t] += sa2[t] * d * (float)(sc2 * i2);
        }
      }
    }
  } else if constexpr (QT == QT_IQ3_XXS) {
    // a unit is one 32-value block: 8 codebook indices (a byte each) and a word of four 7-bit sign codes and the 4-bit
    // scale s; value = d / 4 * (1 + 2 s) * the signed magnitude (zero/kernels/decode.cl:183-478, src/quants.h:220-239)
    const PlanesIQ3XXS pl = planes_iq3xxs(plane_rows, nsb);
    const int ib = hl & 7;
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 3;
      const int e1 = sb * 256 + 32 * ib;
      uint4 a1[TB], a2[TB];
      float sa[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        a1[t] = *(const uint4*)(aq + (size_t)tt * K + e1);
        a2[t] = *(const uint4*)(aq + (size_t)tt * K + e1 + 16);
        sa[t] = asc[(size_t)(e1 >> 5) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const size_t rs = n * nsb + sb;
        const uint2 q = *(const uint2*)(rb + pl.qs + rs * 64 + ib * 8);
        const uint32_t a = *(const uint32_t*)(rb + pl.ss + rs * 32 + ib * 4);
        const int sc = 1 + 2 * (int)(a >> 28);
        const float d = 0.25f * f16_bits_to_f32(*(const unsigned short*)(rb + pl.d + rs * 2));
        uint32_t w[8];
#pragma unroll
        for (int l = 0; l < 4; ++l) {
          const uint32_t s8 = iq3xxs_signs8(a, l);
          const uint32_t qq = l < 2 ? q.x : q.y;
          w[2 * l] = iq3s_signed4(iq3s_grid_lds[(qq >> (16 * (l & 1))) & 0xFFu], s8 & 0xFu);
          w[2 * l + 1] = iq3s_signed4(iq3s_grid_lds[(qq >> (16 * (l & 1) + 8)) & 0xFFu], s8 >> 4);
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int i1 = dot4(w[0], a1[t].x, 0);
          i1 = dot4(w[1], a1[t].y, i1);
          i1 = dot4(w[2], a1[t].z, i1);
          i1 = dot4(w[3], a1[t].w, i1);
          i1 = dot4(w[4], a2[t].x, i1);
          i1 = dot4(w[5], a2[t].y, i1);
          i1 = dot4(w[6], a2[t].z, i1);
          i1 = dot4(w[7], a2[t].w, i1);
          acc[r][t] += sa[t] * d * (float)(sc * i1);
        }
      }
    }
  } else if constexpr (QT == QT_Q3_K) {
    // a unit is one 32-value block: two words of low bit pairs, a word of third bits, two 6-bit scales (one per 16
    // values) out of the superblock's 12-byte header; value = d * (scale - 32) * (bits - 4), the two halves' sums
    // weighted in integers as Q6_K's (zero/kernels/decode.cl:203-222 for the fields, :1000-1003 for the formula)
    const PlanesIQ3S pl = planes_iq3s(plane_rows, nsb);
    const int ib = hl & 7;
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 3;
      const int e1 = sb * 256 + 32 * ib;
      uint4 a1[TB], a2[TB];
      float sa[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        a1[t] = *(const uint4*)(aq + (size_t)tt * K + e1);
        a2[t] = *(const uint4*)(aq + (size_t)tt * K + e1 + 16);
        sa[t] = asc[(size_t)(e1 >> 5) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const size_t rs = n * nsb + sb;
        const uint2 q = *(const uint2*)(rb + pl.qs + rs * 64 + ib * 8);
        const uint32_t H = *(const uint32_t*)(rb + pl.sg + rs * 32 + ib * 4);
        const uint32_t* hp = (const uint32_t*)(rb + pl.hd + rs * 12);
        int sc0, sc1;
        q3k_scales(hp[0], hp[1], hp[2], ib, sc0, sc1);
        const float d = f16_bits_to_f32(*(const unsigned short*)(rb + pl.d + rs * 2));
        uint32_t w[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) w[k] = q3k_vals(k < 4 ? q.x : q.y, H, k);
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int i1 = dot4(w[0], a1[t].x, 0);
          i1 = dot4(w[1], a1[t].y, i1);
          i1 = dot4(w[2], a1[t].z, i1);
          i1 = dot4(w[3], a1[t].w, i1);
          int i2 = dot4(w[4], a2[t].x, 0);
          i2 = dot4(w[5], a2[t].y, i2);
          i2 = dot4(w[6], a2[t].z, i2);
          i2 = dot4(w[7], a2[t].w, i2);
          acc[r][t] += sa[t] * d * (float)(sc0 * i1 + sc1 * i2);
        }
      }
    }
  } else if constexpr (QT == QT_IQ3_S) {
    // a unit is one 32-value block: 8 codebook indices (9 bits: a byte and a bit of the block's ninth-bit byte), 32
    // sign bits, one 4-bit scale s; value = +-(1, 3, ..., 15), sub-scale 1 + 2 s (zero/kernels/decode.cl:400-414)
    const PlanesIQ3S pl = planes_iq3s(plane_rows, nsb);
    const int ib = hl & 7;
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 3;
      const int e1 = sb * 256 + 32 * ib;
      uint4 a1[TB], a2[TB];
      float sa[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        a1[t] = *(const uint4*)(aq + (size_t)tt * K + e1);
        a2[t] = *(const uint4*)(aq + (size_t)tt * K + e1 + 16);
        sa[t] = asc[(size_t)(e1 >> 5) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const size_t rs = n * nsb + sb;
        const uint2 q = *(const uint2*)(rb + pl.qs + rs * 64 + ib * 8);
        const uint32_t sg = *(const uint32_t*)(rb + pl.sg + rs * 32 + ib * 4);
        const uint32_t h9 = rb[pl.hd + rs * 12 + ib];
        const uint32_t scb = rb[pl.hd + rs * 12 + 8 + (ib >> 1)];
        const int sc = 1 + 2 * (int)((scb >> (4 * (ib & 1))) & 0xFu);
        const float d = f16_bits_to_f32(*(const unsigned short*)(rb + pl.d + rs * 2));
        uint32_t w[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const uint32_t idx = (((k < 4 ? q.x : q.y) >> (8 * (k & 3))) & 0xFFu) | (((h9 >> k) & 1u) << 8);
          w[k] = iq3s_signed4(iq3s_grid_lds[idx], (sg >> (4 * k)) & 0xFu);
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int i1 = dot4(w[0], a1[t].x, 0);
          i1 = dot4(w[1], a1[t].y, i1);
          i1 = dot4(w[2], a1[t].z, i1);
          i1 = dot4(w[3], a1[t].w, i1);
          i1 = dot4(w[4], a2[t].x, i1);
          i1 = dot4(w[5], a2[t].y, i1);
          i1 = dot4(w[6], a2[t].z, i1);
          i1 = dot4(w[7], a2[t].w, i1);
          acc[r][t] += sa[t] * d * (float)(sc * i1);
        }
      }
    }
  } else if constexpr (qt_nib16(QT)) {
    const PlanesQ40 pl = planes_q40(plane_rows, nsb);
    const int ib = hl & 7;  // a unit is one 32-block: low nibbles = its elements 0..15, high = 16..31, value by the type's rule (nibble - 8, or a table entry)
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 3;
      const int e1 = sb * 256 + 32 * ib;
      uint4 a1[TB], a2[TB];
      float sa[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        a1[t] = *(const uint4*)(aq + (size_t)tt * K + e1);
        a2[t] = *(const uint4*)(aq + (size_t)tt * K + e1 + 16);
        sa[t] = asc[(size_t)(e1 >> 5) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const uint4 w = *(const uint4*)(rb + pl.qs + n * nsb * 128 + (size_t)u * 16);
        const float d = nib16_scale<QT>(rb + pl.d, n * nsb * 8 + u);
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int i1 = dot4(nib_vals<QT>(ww[0]), a1[t].x, 0);
          i1 = dot4(nib_vals<QT>(ww[1]), a1[t].y, i1);
          i1 = dot4(nib_vals<QT>(ww[2]), a1[t].z, i1);
          i1 = dot4(nib_vals<QT>(ww[3]), a1[t].w, i1);
          i1 = dot4(nib_vals<QT>(ww[0] >> 4), a2[t].x, i1);
          i1 = dot4(nib_vals<QT>(ww[1] >> 4), a2[t].y, i1);
          i1 = dot4(nib_vals<QT>(ww[2] >> 4), a2[t].z, i1);
          i1 = dot4(nib_vals<QT>(ww[3] >> 4), a2[t].w, i1);
          acc[r][t] += sa[t] * d * (float)i1;   // (the 32-block in one conversion, as the reference's gemv: decode.cl:1003)
        }
      }
    }
  } else if constexpr (QT == QT_IQ4_XS) {
    const PlanesIQ4XS pl = planes_iq4xs(plane_rows, nsb);
    const int ib = hl & 7;  // a unit is one 32-block: low nibbles = its elements 0..15, high = 16..31
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 3;
      const int e1 = sb * 256 + 32 * ib;
      uint4 a1[TB], a2[TB];
      float sa[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        a1[t] = *(const uint4*)(aq + (size_t)tt * K + e1);
        a2[t] = *(const uint4*)(aq + (size_t)tt * K + e1 + 16);
        sa[t] = asc[(size_t)(e1 >> 5) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const uint4 w = *(const uint4*)(rb + pl.qs + n * nsb * 128 + (size_t)u * 16);
        const uint2 h = *(const uint2*)(rb + pl.hdr + (n * nsb + sb) * 8);
        const int ls = (int)(((h.y >> (4 * ib)) & 0xFu) | ((((h.x >> 16) >> (2 * ib)) & 3u) << 4)) - 32;
        const float d = f16_bits_to_f32(h.x);
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
        uint32_t w1[4], w2[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          w1[k] = iq4_lookup(ww[k]);
          w2[k] = iq4_lookup(ww[k] >> 4);
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int i1 = dot4(w1[0], a1[t].x, 0);
          i1 = dot4(w1[1], a1[t].y, i1);
          i1 = dot4(w1[2], a1[t].z, i1);
          i1 = dot4(w1[3], a1[t].w, i1);
          i1 = dot4(w2[0], a2[t].x, i1);
          i1 = dot4(w2[1], a2[t].y, i1);
          i1 = dot4(w2[2], a2[t].z, i1);
          i1 = dot4(w2[3], a2[t].w, i1);
          acc[r][t] += sa[t] * d * (float)(ls * i1);
        }
      }
    }
  } else {
    const PlanesQ80 pl = planes_q80(plane_rows, nsb);
    for (int u = hl; u < units; u += 32) {
      const int sb = u >> 4, b = (u >> 1) & 7;
      const int e = u * 16;
      uint4 a[TB];
      float sa[TB];
#pragma unroll
      for (int t = 0; t < TB; ++t) if (t < nt) {
        const int tt = tok[t];
        a[t] = *(const uint4*)(aq + (size_t)tt * K + e);
        sa[t] = asc[(size_t)(e >> 5) * M + tt];
      }
#pragma unroll
      for (int r = 0; r < GROWS; ++r) {
        const size_t n = rows[r];
        const uint8_t* rb = r < SPLIT ? raw : raw2;
        const uint4 w = *(const uint4*)(rb + pl.qs + n * nsb * 256 + (size_t)u * 16);
        const float d = f16_bits_to_f32(*(const unsigned short*)(rb + pl.d + ((n * nsb + sb) * 8 + b) * 2));
#pragma unroll
        for (int t = 0; t < TB; ++t) if (t < nt) {
          int i = dot4(w.x, a[t].x, 0);
          i = dot4(w.y, a[t].y, i);
          i = dot4(w.z, a[t].z, i);
          i = dot4(w.w, a[t].w, i);
          acc[r][t] += sa[t] * d * (float)i;
        }
      }
    }
  }
}

template <int QT, int TB, int GROWS>
__device__ inline void gemv_body(const uint8_t* __restrict__ raw, int N, int K, const signed char* __restrict__ aq,
                                 const float* __restrict__ asc, const short* __restrict__ absum, int M, int T,
                                 float* __restrict__ C, int ldc, int c_off, int accumulate, size_t plane_rows,
                                 float softcap = 0.0f) {
  const int hl = threadIdx.x & 31;
  const int hw = (int)((blockIdx.x * blockDim.x + threadIdx.x) >> 5);
  const int r0 = hw * GROWS;
  if (r0 >= N) return;
  float acc[GROWS][TB];
  size_t rows[GROWS];
  int tok[TB];
#pragma unroll
  for (int r = 0; r < GROWS; ++r) {
    rows[r] = (size_t)min(r0 + r, N - 1);
#pragma unroll
    for (int t = 0; t < TB; ++t) acc[r][t] = 0.0f;
  }
#pragma unroll
  for (int t = 0; t < TB; ++t) tok[t] = t < T ? t : 0;
  gemv_acc<QT, TB, GROWS>(raw, plane_rows, rows, K, tok, aq, asc, absum, M, hl, acc);

#pragma unroll
  for (int r = 0; r < GROWS; ++r)
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      const float v = head_out(half_wave_sum(acc[r][t]), softcap);
      const int n = r0 + r;
      if (hl == 0 && n < N && t < T) {
        float* cp = C + (size_t)t * ldc + c_off + n;
        *cp = accumulate ? *cp + v : v;
      }
    }
}

// gemv_v: one token, activations read straight from global memory (the fallback when a chunk's activations do not
// fit LDS).  Arguments as the reference's gemv_v (zero/kernels/decode.cl:1353); `tabs` (its codebook tables) is
// unused by these three types.  grid: ceil(N / GROWS) half waves in work-groups of 256.
#define GEMV_INST(QT, GROWS)                                                                                         \
  extern "C" __global__ __launch_bounds__(256) void gemv_v__QT##QT##_GROWS##GROWS(                                      \
      const uint8_t* raw, int N, int K, const uint32_t* tabs, const signed char* aq, const float* asc,               \
      const short* absum, int M, float* C, int c_off, int accumulate, float softcap) {                                \
    grid_init<QT>(tabs);                                                                                           \
    gemv_body<QT, 1, GROWS>(raw, N, K, aq, asc, absum, M, 1, C, 0, c_off, accumulate, (size_t)N, softcap);           \
  }

// gemv_mt_v: T = TB tokens (reference zero/kernels/decode.cl:1426).
#define GEMV_MT_INST(QT, GROWS, TB)                                                                                  \
  extern "C" __global__ __launch_bounds__(256) void gemv_mt_v__QT##QT##_GROWS##GROWS##_TB##TB(                          \
      const uint8_t* raw, int N, int K, const uint32_t* tabs, const signed char* aq, const float* asc,               \
      const short* absum, int M, int T, float* C, int ldc, int c_off, int accumulate, float softcap) {                \
    grid_init<QT>(tabs);                                                                                           \
    gemv_body<QT, TB, GROWS>(raw, N, K, aq, asc, absum, M, T, C, ldc, c_off, accumulate, (size_t)N, softcap);        \
  }

#define GEMV_ALL(QT)                                                                                                 \
  GEMV_INST(QT, 1) GEMV_INST(QT, 2) GEMV_INST(QT, 4)                                                                  \
  GEMV_MT_INST(QT, 1, 2) GEMV_MT_INST(QT, 1, 3) GEMV_MT_INST(QT, 1, 4) GEMV_MT_INST(QT, 1, 5)                         \
  GEMV_MT_INST(QT, 1, 6) GEMV_MT_INST(QT, 1, 7) GEMV_MT_INST(QT, 1, 8)                                                \
  GEMV_MT_INST(QT, 2, 2) GEMV_MT_INST(QT, 2, 3) GEMV_MT_INST(QT, 2, 4) GEMV_MT_INST(QT, 2, 5)                         \
  GEMV_MT_INST(QT, 2, 6) GEMV_MT_INST(QT, 2, 7) GEMV_MT_INST(QT, 2, 8)

GEMV_ALL(8)
GEMV_ALL(12)
GEMV_ALL(13)
GEMV_ALL(14)
GEMV_ALL(23)
GEMV_ALL(2)
GEMV_ALL(18)
GEMV_ALL(11)
GEMV_ALL(20)
GEMV_ALL(39)
GEMV_ALL(21)

// ---- the experts of a pass of a few tokens (the reference's per-tile kernels moe_gateup_q / moe_down_q,
// zero/kernels/decode.cl, launched by zero/engine_moe.h:196-262 with tiles of TM = 1, 2, 4 or 8 slots for 1-8 tokens):
// the matrix-vector form above on the rows of one expert.  A tile of the list = (expert, first slot, slots <= TM), made
// by moe_route1 (one token: its NU experts are the tiles), moe_route_small or moe_scan.
// grid (ceil(rows / GROWS) half waves in work-groups of 256, tile work-groups: y, y + gridDim.y, ...).

// moe_gateup_q: h[slot][f] = silu(gate) * up for the tile's slots, gate and up from the two expert tensors' rows
// [NE][F][K]; slot r reads token row stok[r].  Arguments as the reference's (rg, ru, F, K, tabs, aq, asc, M, tiles, stok,
// h) plus absum (the 16-value sums the Q4_K / Q5_K min term takes) and NE.
template <int QT, int TM, int GROWS>
__device__ inline void moe_gateup_rows(const uint8_t* __restrict__ rg, const uint8_t* __restrict__ ru, int F, int K,
                                       const signed char* __restrict__ aq, const float* __restrict__ asc,
                                       const short* __restrict__ absum, int M, const int* __restrict__ tiles,
                                       const int* __restrict__ stok, float* __restrict__ h, int NE) {
  const int hl = threadIdx.x & 31;
  const int hw = (int)((blockIdx.x * blockDim.x + threadIdx.x) >> 5);
  const int f0 = hw * GROWS;
  if (f0 >= F) return;
  const int nt = tiles[0];
  for (int ti = blockIdx.y; ti < nt; ti += gridDim.y) {
    const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = min(tiles[3 + 3 * ti], TM);
    float ag[GROWS][TM], au[GROWS][TM];
    size_t rows[GROWS];
    int tok[TM];
#pragma unroll
    for (int r = 0; r < GROWS; ++r) {
      rows[r] = (size_t)e * F + min(f0 + r, F - 1);
#pragma unroll
      for (int t = 0; t < TM; ++t) ag[r][t] = au[r][t] = 0.0f;
    }
#pragma unroll
    for (int t = 0; t < TM; ++t) tok[t] = stok[r0 + min(t, nr - 1)];
    gemv_acc<QT, TM, GROWS>(rg, (size_t)NE * F, rows, K, tok, aq, asc, absum, M, hl, ag, nr);
    gemv_acc<QT, TM, GROWS>(ru, (size_t)NE * F, rows, K, tok, aq, asc, absum, M, hl, au, nr);
#pragma unroll
    for (int r = 0; r < GROWS; ++r)
#pragma unroll
      for (int t = 0; t < TM; ++t) {
        if (t >= nr) continue;  // (the same for the whole wave)
        const float g = half_wave_sum(ag[r][t]), u = half_wave_sum(au[r][t]);
        if (hl == 0 && f0 + r < F) h[(size_t)(r0 + t) * F + f0 + r] = g / (1.0f + __expf(-g)) * u;
      }
  }
}

// moe_down_q: y[slot][n] = swt[slot] * (Wd[expert][n] . hq[slot]) for the tile's slots; the expert tensor's rows
// [NE][N][K], hq / hsc / hbs the expert inputs as moe_quant_sums leaves them (row stride S slots).  Arguments as the
// reference's (raw, N, K, tabs, hq, hsc, S, tiles, swt, y) plus hbs and NE.
template <int QT, int TM, int GROWS>
__device__ inline void moe_down_rows(const uint8_t* __restrict__ raw, int N, int K, const signed char* __restrict__ hq,
                                     const float* __restrict__ hsc, const short* __restrict__ hbs, int S,
                                     const int* __restrict__ tiles, const float* __restrict__ swt, float* __restrict__ y,
                                     int NE) {
  const int hl = threadIdx.x & 31;
  const int hw = (int)((blockIdx.x * blockDim.x + threadIdx.x) >> 5);
  const int n0 = hw * GROWS;
  if (n0 >= N) return;
  const int nt = tiles[0];
  for (int ti = blockIdx.y; ti < nt; ti += gridDim.y) {
    const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = min(tiles[3 + 3 * ti], TM);
    float acc[GROWS][TM];
    size_t rows[GROWS];
    int tok[TM];
#pragma unroll
    for (int r = 0; r < GROWS; ++r) {
      rows[r] = (size_t)e * N + min(n0 + r, N - 1);
#pragma unroll
      for (int t = 0; t < TM; ++t) acc[r][t] = 0.0f;
    }
#pragma unroll
    for (int t = 0; t < TM; ++t) tok[t] = r0 + min(t, nr - 1);
    gemv_acc<QT, TM, GROWS>(raw, (size_t)NE * N, rows, K, tok, hq, hsc, hbs, S, hl, acc, nr);
#pragma unroll
    for (int r = 0; r < GROWS; ++r)
#pragma unroll
      for (int t = 0; t < TM; ++t) {
        if (t >= nr) continue;
        const float v = half_wave_sum(acc[r][t]);
        if (hl == 0 && n0 + r < N) y[(size_t)(r0 + t) * N + n0 + r] = swt[r0 + t] * v;
      }
  }
}

// moe_gateup_q -DQUANT: the same with the expert inputs' quantization (moe_quant_sums) done on the way out: a
// work-group's 8 half waves take 4 rows each, one 32-block of h per slot, which the first half wave quantizes as
// quant_store16 does -- amax over the block, q = rte(v * (127 / amax)), scale amax / 127, the sums of 16 -- and stores
// next to the f32 values: hq [S][F], hsc [F/32][S], hbs [F/16][S].  One launch less in a pass of one or two tokens.
// ROUTE (up to 8 tokens, one-slot tiles, grid.y = T * NU): the work-group routes the tokens itself -- wave w token w, as
// moe_route_small does, every work-group the same list -- and takes the pair whose slot is its blockIdx.y; the first
// work-group writes the lists out for the down kernel.  No routing launch at all.
struct MoeRouteArgs {
  const float* logits;
  float *sgate, *swt, *wts;
  int *tiles_out, *stok_out, *inv, *ids;
  int NU, ldl, T;
};
template <int QT, int TM, bool ROUTE = false>
__device__ inline void moe_gateup_quant_rows(const uint8_t* __restrict__ rg, const uint8_t* __restrict__ ru, int F, int K,
                                             const signed char* __restrict__ aq, const float* __restrict__ asc,
                                             const short* __restrict__ absum, int M, const int* tiles, const int* stok,
                                             float* __restrict__ h, int NE, int S, signed char* __restrict__ hq,
                                             float* __restrict__ hsc, short* __restrict__ hbs,
                                             MoeRouteArgs ra = MoeRouteArgs()) {
  constexpr int GR = 2;  // rows of each matrix per half wave: 16 half waves (512 threads) make the 32 rows
  __shared__ float hs[TM][32];
  __shared__ __attribute__((aligned(16))) int sid[ROUTE ? 512 : 4];
  __shared__ float sw[ROUTE ? 512 : 1];
  __shared__ int s_et[2];  // this work-group's pair: expert, token
  if constexpr (ROUTE) {
    const int lane = threadIdx.x & 63, tw = threadIdx.x >> 6, NU = ra.NU, n = ra.T * NU;
    const bool first = blockIdx.x == 0 && blockIdx.y == 0;
    if (tw < ra.T) {
      const float* lg = ra.logits + (size_t)tw * ra.ldl;
      int sel;
      float wt;
      route_one_token(lg, NE, NU, lane, sel, wt);
      if (lane < NU) {
        sid[tw * NU + lane] = sel;
        sw[tw * NU + lane] = wt;
        if (first) { ra.ids[tw * NU + lane] = sel; ra.wts[tw * NU + lane] = wt; }
      }
      if (first && lane == 0 && ra.sgate) ra.sgate[tw] = ra.ldl > NE ? 1.0f / (1.0f + expf(-lg[NE])) : 0.0f;
    }
    if ((int)threadIdx.x >= n) sid[threadIdx.x] = 0x7FFFFFFF;  // (an expert no pair has: the list is read in fours)
    __syncthreads();
    const int i = threadIdx.x;
    if (i < n) {  // slot of pair i = pairs of lower experts + earlier pairs of its own (moe_route_small's layout)
      const int e = sid[i];
      int slot = 0;
      for (int j = 0; j < ((n + 3) & ~3); j += 4) {
        const int4 q = *(const int4*)&sid[j];
        const int ej[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) slot += (ej[c] < e || (ej[c] == e && j + c < i)) ? 1 : 0;
      }
      if (slot == (int)blockIdx.y) { s_et[0] = e; s_et[1] = i / NU; }
      if (first) {
        ra.tiles_out[1 + 3 * slot] = e;
        ra.tiles_out[2 + 3 * slot] = slot;
        ra.tiles_out[3 + 3 * slot] = 1;
        ra.stok_out[slot] = i / NU;
        ra.swt[slot] = sw[i];
        ra.inv[i] = slot;
        if (i == 0) ra.tiles_out[0] = n;
      }
    }
    __syncthreads();
  }
  const int hl = threadIdx.x & 31, w = threadIdx.x >> 5;
  const int fb = blockIdx.x * 32, f0 = fb + w * GR;  // (F is a multiple of 32: every row of the block exists)
  const int nt = ROUTE ? (int)blockIdx.y + 1 : tiles[0];  // (ROUTE: exactly the one tile)
  for (int ti = blockIdx.y; ROUTE || TM == 1 || ti < nt; ti += gridDim.y) {
    // (one-slot tiles: tile ti is slot ti, so the tile's expert and the slot's token are read beside the tile count,
    //  one memory latency instead of three in a row; an index past the lists' used part reads what lies there and is
    //  dropped by the test below)
    const int e = ROUTE ? s_et[0] : tiles[1 + 3 * ti], r0 = ROUTE || TM == 1 ? ti : tiles[2 + 3 * ti],
              nr = ROUTE || TM == 1 ? 1 : min(tiles[3 + 3 * ti], TM);
    const int tok1 = ROUTE ? s_et[1] : TM == 1 ? stok[min(ti, S - 1)] : 0;
    if (ti >= nt) break;
    float a[2 * GR][TM];  // [0, GR): gate rows, [GR, 2 GR): the same rows of up
    size_t rows[2 * GR];
    int tok[TM];
#pragma unroll
    for (int r = 0; r < 2 * GR; ++r) {
      rows[r] = (size_t)e * F + f0 + (r % GR);
#pragma unroll
      for (int t = 0; t < TM; ++t) a[r][t] = 0.0f;
    }
#pragma unroll
    for (int t = 0; t < TM; ++t) tok[t] = ROUTE || TM == 1 ? tok1 : stok[r0 + min(t, nr - 1)];
    gemv_acc<QT, TM, 2 * GR, GR>(rg, (size_t)NE * F, rows, K, tok, aq, asc, absum, M, hl, a, nr, ru);
#pragma unroll
    for (int r = 0; r < GR; ++r)
#pragma unroll
      for (int t = 0; t < TM; ++t) {
        if (t >= nr) continue;  // (the same for the whole work-group)
        const float g = half_wave_sum(a[r][t]), u = half_wave_sum(a[GR + r][t]);
        if (hl == 0) hs[t][w * GR + r] = g / (1.0f + __expf(-g)) * u;
      }
    __syncthreads();
    if (w == 0) {
#pragma unroll
      for (int t = 0; t < TM; ++t) {
        if (t >= nr) continue;
        const float v = hs[t][hl];
        float amax = fabsf(v);
#pragma unroll
        for (int o = 16; o >= 1; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
        const int q = __float2int_rn(__fmul_rn(v, inv));
        int sm = q;
#pragma unroll
        for (int o = 8; o >= 1; o >>= 1) sm += __shfl_xor(sm, o, 64);  // the 16 lanes of a half block
        const size_t slot = (size_t)(r0 + t);
        h[slot * F + fb + hl] = v;
        hq[slot * F + fb + hl] = (signed char)q;
        if (hl == 0) hsc[(size_t)(fb >> 5) * S + slot] = amax / 127.0f;
        if ((hl & 15) == 0) hbs[(size_t)((fb >> 4) + (hl >> 4)) * S + slot] = (short)sm;
      }
    }
    __syncthreads();
  }
}

// moe_down1_q: the down projections of a pass whose tiles hold one slot each (slot s is tile s) and their sum in one
// kernel: x[t][n] += sum over k (in order) of swt[s] * (Wd[expert of s][n] . hq[s]), s = inv[t * NU + k] -- moe_down_q
// and moe_combine without the y rows in between; the same sums in the same order.  grid (ceil(N / GROWS) work-groups
// of 256, tokens); NU <= 64.
template <int QT, int GROWS>
__device__ inline void moe_down1_rows(const uint8_t* __restrict__ raw, int N, int K, const signed char* __restrict__ hq,
                                      const float* __restrict__ hsc, const short* __restrict__ hbs, int S,
                                      const int* __restrict__ tiles, const float* __restrict__ swt, float* __restrict__ x,
                                      const int* __restrict__ inv, int NU, int NE) {
  // a work-group takes GROWS rows of x[t]; its 8 half waves take the token's experts k = w, w + 8, ... side by side
  // (one after the other a token's 8 short rows were 8 memory latencies), and the weighted products meet in LDS
  __shared__ float part[64][GROWS];
  const int hl = threadIdx.x & 31, w = threadIdx.x >> 5;
  const int n0 = blockIdx.x * GROWS, t = blockIdx.y;
  for (int k = w; k < NU; k += 8) {
    const int sl = inv[t * NU + k], e = tiles[1 + 3 * sl];
    float acc[GROWS][1];
    size_t rows[GROWS];
    const int tok[1] = {sl};
#pragma unroll
    for (int r = 0; r < GROWS; ++r) {
      rows[r] = (size_t)e * N + min(n0 + r, N - 1);
      acc[r][0] = 0.0f;
    }
    gemv_acc<QT, 1, GROWS>(raw, (size_t)NE * N, rows, K, tok, hq, hsc, hbs, S, hl, acc);
    const float wt = swt[sl];
#pragma unroll
    for (int r = 0; r < GROWS; ++r) {
      const float v = half_wave_sum(acc[r][0]);
      if (hl == 0) part[k][r] = wt * v;
    }
  }
  __syncthreads();
  if (threadIdx.x < GROWS && n0 + (int)threadIdx.x < N) {
    float v = 0.0f;
    for (int k = 0; k < NU; ++k) v += part[k][threadIdx.x];
    x[(size_t)t * N + n0 + threadIdx.x] += v;
  }
}

#define MOE_DECODE_FUSED_INST(QT)                                                                                    \
  extern "C" __global__ __launch_bounds__(512) void moe_gateup_q__QT##QT##_GROWS4_TM1_QUANT1(                         \
      const uint8_t* rg, const uint8_t* ru, int F, int K, const uint32_t* tabs, const signed char* aq, const float* asc, \
      int M, const int* tiles, const int* stok, float* h, const short* absum, int S, signed char* hq, float* hsc,     \
      short* hbs, int NE) {                                                                                           \
    grid_init<QT>(tabs);                                                                                           \
    moe_gateup_quant_rows<QT, 1>(rg, ru, F, K, aq, asc, absum, M, tiles, stok, h, NE, S, hq, hsc, hbs);              \
  }                                                                                                                   \
  extern "C" __global__ __launch_bounds__(512) void moe_gateup_q__QT##QT##_GROWS4_TM2_QUANT1(                         \
      const uint8_t* rg, const uint8_t* ru, int F, int K, const uint32_t* tabs, const signed char* aq, const float* asc, \
      int M, const int* tiles, const int* stok, float* h, const short* absum, int S, signed char* hq, float* hsc,     \
      short* hbs, int NE) {                                                                                           \
    grid_init<QT>(tabs);                                                                                           \
    moe_gateup_quant_rows<QT, 2>(rg, ru, F, K, aq, asc, absum, M, tiles, stok, h, NE, S, hq, hsc, hbs);              \
  }                                                                                                                   \
  extern "C" __global__ __launch_bounds__(512) void moe_gateup_q__QT##QT##_GROWS4_TM1_QUANT1_ROUTE1(                  \
      const uint8_t* rg, const uint8_t* ru, int F, int K, const uint32_t* tabs, const signed char* aq, const float* asc, \
      int M, int* tiles, int* stok, float* h, const short* absum, int S, signed char* hq, float* hsc, short* hbs,     \
      const float* logits, float* sgate, float* swt, int* inv, int NU, int ldl, int T, int* ids, float* wts, int NE) { \
    grid_init<QT>(tabs);                                                                                           \
    MoeRouteArgs ra;                                                                                                  \
    ra.logits = logits; ra.sgate = sgate; ra.swt = swt; ra.tiles_out = tiles; ra.stok_out = stok; ra.inv = inv;       \
    ra.NU = NU; ra.ldl = ldl; ra.T = T; ra.ids = ids; ra.wts = wts;                                                   \
    moe_gateup_quant_rows<QT, 1, true>(rg, ru, F, K, aq, asc, absum, M, tiles, stok, h, NE, S, hq, hsc, hbs, ra);     \
  }                                                                                                                   \
  extern "C" __global__ __launch_bounds__(256) void moe_down1_q__QT##QT##_GROWS4(                                     \
      const uint8_t* raw, int N, int K, const uint32_t* tabs, const signed char* hq, const float* hsc, int S,         \
      const int* tiles, const float* swt, float* x, const short* hbs, const int* inv, int NU, int NE) {              \
    grid_init<QT>(tabs);                                                                                           \
    moe_down1_rows<QT, 4>(raw, N, K, hq, hsc, hbs, S, tiles, swt, x, inv, NU, NE);                                   \
  }
MOE_DECODE_FUSED_INST(8)
MOE_DECODE_FUSED_INST(12)
MOE_DECODE_FUSED_INST(13)
MOE_DECODE_FUSED_INST(14)
MOE_DECODE_FUSED_INST(23)
MOE_DECODE_FUSED_INST(2)
MOE_DECODE_FUSED_INST(18)
MOE_DECODE_FUSED_INST(11)
MOE_DECODE_FUSED_INST(20)
MOE_DECODE_FUSED_INST(39)
MOE_DECODE_FUSED_INST(21)

#define MOE_DECODE_INST(QT, TM)                                                                                      \
  extern "C" __global__ __launch_bounds__(256) void moe_gateup_q__QT##QT##_GROWS2_TM##TM(                             \
      const uint8_t* rg, const uint8_t* ru, int F, int K, const uint32_t* tabs, const signed char* aq, const float* asc, \
      int M, const int* tiles, const int* stok, float* h, const short* absum, int NE) {                              \
    grid_init<QT>(tabs);                                                                                           \
    moe_gateup_rows<QT, TM, 2>(rg, ru, F, K, aq, asc, absum, M, tiles, stok, h, NE);                                 \
  }                                                                                                                   \
  extern "C" __global__ __launch_bounds__(256) void moe_down_q__QT##QT##_GROWS2_TM##TM(                               \
      const uint8_t* raw, int N, int K, const uint32_t* tabs, const signed char* hq, const float* hsc, int S,         \
      const int* tiles, const float* swt, float* y, const short* hbs, int NE) {                                      \
    grid_init<QT>(tabs);                                                                                           \
    moe_down_rows<QT, TM, 2>(raw, N, K, hq, hsc, hbs, S, tiles, swt, y, NE);                                         \
  }
#define MOE_DECODE_ALL(QT) MOE_DECODE_INST(QT, 1) MOE_DECODE_INST(QT, 2) MOE_DECODE_INST(QT, 4) MOE_DECODE_INST(QT, 8)
MOE_DECODE_ALL(8)
MOE_DECODE_ALL(12)
MOE_DECODE_ALL(13)
MOE_DECODE_ALL(14)
MOE_DECODE_ALL(23)
MOE_DECODE_ALL(2)
MOE_DECODE_ALL(18)
MOE_DECODE_ALL(11)
MOE_DECODE_ALL(20)
MOE_DECODE_ALL(39)
MOE_DECODE_ALL(21)

// expand_iq3s: the IQ3_S planes of `rows` rows to Q6_K planes of the same rows, value for value -- the same f16 d, the
// int8 sub-scale 1 + 2 s for both 16-value halves of a block, q = value + 32 in six bits -- for the prefill GEMM and
// the expert-tile GEMM, which run their Q6_K kernels on the result (the place of the reference's decode pass in front
// of its GEMM, zero/engine.h:1205-1250 with zero/kernels/decode.cl:183-478).  Thread (superblock, n, j) makes the words
// ql[64 n + 4 j ..], ql[64 n + 32 + 4 j ..] and qh[32 n + 4 j ..]: the values 4 j .. 4 j + 3 of blocks 4 n .. 4 n + 3,
// one codebook entry per block.  grid: ceil(rows * nsb / 16) work-groups of 256 (16 threads a superblock).
extern "C" __global__ __launch_bounds__(256) void expand_iq3s(const uint8_t* __restrict__ raw, uint8_t* __restrict__ out,
                                                              const uint32_t* __restrict__ tabs, int rows, int nsb) {
  iq3s_grid_init(tabs);
  const size_t total = (size_t)rows * nsb;
  const size_t rs = (size_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (rs >= total) return;
  const PlanesIQ3S pi = planes_iq3s((size_t)rows, nsb);
  const PlanesQ6K po = planes_q6k((size_t)rows, nsb);
  const int n = (threadIdx.x >> 3) & 1, j = threadIdx.x & 7;
  const uint32_t h9 = *(const uint32_t*)(raw + pi.hd + rs * 12 + 4 * n);  // the ninth bits of blocks 4 n .. 4 n + 3
  uint32_t q[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int ib = 4 * n + k;
    const uint32_t idx = raw[pi.qs + rs * 64 + ib * 8 + j] | ((((h9 >> (8 * k)) >> j) & 1u) << 8);
    const uint32_t s4 = ((uint32_t)raw[pi.sg + rs * 32 + ib * 4 + (j >> 1)] >> (4 * (j & 1))) & 0xFu;
    const uint32_t v = iq3s_signed4(iq3s_grid_lds[idx], s4);
    q[k] = ((v & 0x7F7F7F7Fu) + 0x20202020u) ^ (v & 0x80808080u);  // value + 32 in every byte, no carry between bytes
  }
  const uint32_t lo = 0x0F0F0F0Fu, two = 0x03030303u;
  *(uint32_t*)(out + po.ql + rs * 128 + 64 * n + 4 * j) = (q[0] & lo) | ((q[2] & lo) << 4);
  *(uint32_t*)(out + po.ql + rs * 128 + 64 * n + 32 + 4 * j) = (q[1] & lo) | ((q[3] & lo) << 4);
  *(uint32_t*)(out + po.qh + rs * 64 + 32 * n + 4 * j) =
      ((q[0] >> 4) & two) | (((q[1] >> 4) & two) << 2) | (((q[2] >> 4) & two) << 4) | (((q[3] >> 4) & two) << 6);
  if (n == 0 && j < 4) {  // sub-scales 4 j .. 4 j + 3: blocks 2 j and 2 j + 1, each for both of its halves
    const uint32_t sb = raw[pi.hd + rs * 12 + 8 + j];
    const uint32_t s0 = 1 + 2 * (sb & 0xFu), s1 = 1 + 2 * (sb >> 4);
    *(uint32_t*)(out + po.sc + rs * 16 + 4 * j) = s0 | (s0 << 8) | (s1 << 16) | (s1 << 24);
  }
  if (n == 1 && j == 0) *(unsigned short*)(out + po.d + rs * 2) = *(const unsigned short*)(raw + pi.d + rs * 2);
}

// expand_q3k: the Q3_K planes of `rows` rows to Q6_K planes of the same rows, value for value -- the same f16 d, the
// 6-bit scales - 32 as the int8 sub-scales, q = value + 32 in six bits -- for the prefill GEMM and the expert-tile GEMM,
// as expand_iq3s.  Thread (superblock, n, j) makes the words ql[64 n + 4 j ..], ql[64 n + 32 + 4 j ..] and
// qh[32 n + 4 j ..]: the values 4 j .. 4 j + 3 of blocks 4 n .. 4 n + 3.  grid: ceil(rows * nsb / 16) work-groups of 256.
extern "C" __global__ __launch_bounds__(256) void expand_q3k(const uint8_t* __restrict__ raw, uint8_t* __restrict__ out, int rows,
                                                             int nsb) {
  const size_t total = (size_t)rows * nsb;
  const size_t rs = (size_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (rs >= total) return;
  const PlanesIQ3S pi = planes_iq3s((size_t)rows, nsb);
  const PlanesQ6K po = planes_q6k((size_t)rows, nsb);
  const int n = (threadIdx.x >> 3) & 1, j = threadIdx.x & 7;
  uint32_t q[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int ib = 4 * n + k;
    const uint32_t D = *(const uint32_t*)(raw + pi.qs + rs * 64 + ib * 8 + 4 * (j >> 2));
    const uint32_t H = *(const uint32_t*)(raw + pi.sg + rs * 32 + ib * 4);
    const uint32_t v = q3k_vals(D, H, j);
    q[k] = ((v & 0x7F7F7F7Fu) + 0x20202020u) ^ (v & 0x80808080u);  // value + 32 in every byte, no carry between bytes
  }
  const uint32_t lo = 0x0F0F0F0Fu, two = 0x03030303u;
  *(uint32_t*)(out + po.ql + rs * 128 + 64 * n + 4 * j) = (q[0] & lo) | ((q[2] & lo) << 4);
  *(uint32_t*)(out + po.ql + rs * 128 + 64 * n + 32 + 4 * j) = (q[1] & lo) | ((q[3] & lo) << 4);
  *(uint32_t*)(out + po.qh + rs * 64 + 32 * n + 4 * j) =
      ((q[0] >> 4) & two) | (((q[1] >> 4) & two) << 2) | (((q[2] >> 4) & two) << 4) | (((q[3] >> 4) & two) << 6);
  if (n == 0) {  // sub-scales 2 j, 2 j + 1: block j's two
    const uint32_t* hp = (const uint32_t*)(raw + pi.hd + rs * 12);
    int sc0, sc1;
    q3k_scales(hp[0], hp[1], hp[2], j, sc0, sc1);
    *(unsigned short*)(out + po.sc + rs * 16 + 2 * j) = (unsigned short)((uint32_t)(sc0 & 0xFF) | ((uint32_t)(sc1 & 0xFF) << 8));
  }
  if (n == 1 && j == 0) *(unsigned short*)(out + po.d + rs * 2) = *(const unsigned short*)(raw + pi.d + rs * 2);
}

// expand_iq3xxs: the IQ3_XXS planes of `rows` rows to Q6_K planes of the same rows that hold HALF the values -- the
// magnitudes are even, so q = value / 2 + 32 fits six bits; the int8 sub-scale 1 + 2 s for both halves of a block; and
// d / 4, which an f16 cannot always hold, as d unchanged: the Q6_K GEMM kernels that run on these planes (-DHD, -DHDS,
// -DHDT) halve their factor of d -- as expand_iq3s.  Thread (superblock, n, j) makes the words ql[64 n + 4 j ..],
// ql[64 n + 32 + 4 j ..] and qh[32 n + 4 j ..]: the values 4 j .. 4 j + 3 of blocks 4 n .. 4 n + 3, one codebook entry per
// block.  grid: ceil(rows * nsb / 16) work-groups of 256.
extern "C" __global__ __launch_bounds__(256) void expand_iq3xxs(const uint8_t* __restrict__ raw, uint8_t* __restrict__ out,
                                                                const uint32_t* __restrict__ tabs, int rows, int nsb) {
  grid_init<QT_IQ3_XXS>(tabs);
  const size_t total = (size_t)rows * nsb;
  const size_t rs = (size_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (rs >= total) return;
  const PlanesIQ3XXS pi = planes_iq3xxs((size_t)rows, nsb);
  const PlanesQ6K po = planes_q6k((size_t)rows, nsb);
  const int n = (threadIdx.x >> 3) & 1, j = threadIdx.x & 7;
  uint32_t q[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int ib = 4 * n + k;
    const uint32_t a = *(const uint32_t*)(raw + pi.ss + rs * 32 + ib * 4);
    const uint32_t s4 = (iq3xxs_signs8(a, j >> 1) >> (4 * (j & 1))) & 0xFu;
    const uint32_t v = iq3s_signed4(iq3s_grid_lds[raw[pi.qs + rs * 64 + ib * 8 + j]] >> 1, s4);  // (magnitudes halved: 2 .. 31)
    q[k] = ((v & 0x7F7F7F7Fu) + 0x20202020u) ^ (v & 0x80808080u);  // value + 32 in every byte, no carry between bytes
  }
  const uint32_t lo = 0x0F0F0F0Fu, two = 0x03030303u;
  *(uint32_t*)(out + po.ql + rs * 128 + 64 * n + 4 * j) = (q[0] & lo) | ((q[2] & lo) << 4);
  *(uint32_t*)(out + po.ql + rs * 128 + 64 * n + 32 + 4 * j) = (q[1] & lo) | ((q[3] & lo) << 4);
  *(uint32_t*)(out + po.qh + rs * 64 + 32 * n + 4 * j) =
      ((q[0] >> 4) & two) | (((q[1] >> 4) & two) << 2) | (((q[2] >> 4) & two) << 4) | (((q[3] >> 4) & two) << 6);
  if (n == 0) {  // sub-scales 2 j, 2 j + 1: block j's, the same for both of its halves
    const uint32_t sc = 1u + 2u * (*(const uint32_t*)(raw + pi.ss + rs * 32 + j * 4) >> 28);
    *(unsigned short*)(out + po.sc + rs * 16 + 2 * j) = (unsigned short)(sc | (sc << 8));
  }
  if (n == 1 && j == 0) *(unsigned short*)(out + po.d + rs * 2) = *(const unsigned short*)(raw + pi.d + rs * 2);
}
