// "gemm" module: the prefill GEMM  C[m][c_off + n] (=, +=, silu(C) *) sum_k A[m][k] W[n][k]  on int8 MFMA, for dense
// matrices and for the expert-grouped tiles of a mixture-of-experts layer.
//
// Arithmetic (reference zero/kernels/gemm.cl:439-488, the per-32 activation scale form): every 32-block b of K gives
// an exact int32 sum I[m][n][b] (v_mfma_i32_32x32x32_i8, accumulator cleared per block), then in f32
//   Q8_0 : res += (sa[m][b] * d[n][b]) * (float)I
//   Q4_K : res += (sa[m][b] * (d[n] * sc[n][b])) * (float)I  -  (sa[m][b] * (float)S[m][b]) * (dmin[n] * mn[n][b])
//   Q5_K : as Q4_K (values 0..31)
//   IQ4_XS: res += (sa[m][b] * (d[n] * ls[n][b])) * (float)I      (ls: the block's 6-bit scale - 32)
// with S the sum of the block's 32 int8 activations.  Blocks are added in K order.
//
// The scheme needs one f32 scale per (token, weight row, block), so the vector ALU, not the matrix pipe, bounds it.
// The tuned kernel therefore leaves the ALU two instructions per product and block -- int -> float and one fma -- and
// moves the rest to the matrix pipe, which has cycles to spare:
//   * the scale tile P[m][n] = sa[m][b] * ws[n][b] is an outer product: v_mfma_f32_32x32x1_2b_f32 makes two 32 x 32
//     tiles of exact f32 products per instruction;
//   * the Q4_K min term  - sum_b U[m][b] V[n][b]  (U = sa * S, V = dmin * mn) is a rank-(K/32) f32 product:
//     v_mfma_f32_32x32x2_f32 adds two blocks per instruction straight into the result accumulators.
// Tiling: a work-group of 256 threads (4 waves, 2 x 2) computes 128 tokens x 128 weight rows, a wave 64 x 64 as 2 x 2
// MFMA tiles.  K advances in half superblocks (128 values): tokens' int8 values and weight rows decoded to int8 are
// staged in LDS with a 16-byte row pad (conflict-free 128-bit reads) next to the four scale vectors of each block;
// the next step's global loads are in flight while the current step is computed.  The A operand is the token tile
// and B the weight tile, so a lane owns one weight row n and writes 128-byte runs of C.  Work-groups are numbered so
// that the 64 that run together on one XCD form an 8 x 8 block of tiles and share their operands in that XCD's L2.
#include "common.h"
#include "quant.h"

#define BM 128
#define BN 128
#define BK 128
#define LDS_PAD 16

#include "gemm_simple.inc"

struct alignas(16) Gemm2Lds {
  alignas(16) uint8_t act[BM][BK + LDS_PAD];
  alignas(16) uint8_t wq[BN][BK + LDS_PAD];
  float sa[4][BM];   // activation scale of the step's 4 blocks
  float u[4][BM];    // sa * S (Q4_K)
  float ws[4][BN];   // weight scale d * sc (Q8_0: d)
  float v[4][BN];    // -(dmin * mn) (Q4_K)
  int rowmap[BM];
};

// The (tile, row chunk) a work-group of a tile kernel takes, nc row chunks a tile, grid (nc, tile work-groups) with the
// tile work-groups at least the tiles there are, and a multiple of 8.  The XCDs take work-groups in turn (linear id % 8) and each has its own L2, so the
// tile list, which is sorted by expert, is cut into 8 runs, one per XCD, and the work-groups of an XCD walk their run
// in groups of 4 tiles, row chunk by row chunk: four neighbours read the same rows of an expert (mostly: an expert of
// 256 slots has 4 or 5 tiles), and the 4 nc work-groups of a group the same slots' activations, out of one L2.  Every
// tile and chunk is taken exactly once; work-groups beyond their XCD's run do nothing (false).
__device__ inline bool moe_tile_of(int nt, int nc, int& ti, int& chunk) {
  if (gridDim.y & 7) {  // (a launch of another shape: work-group (x, y) takes chunk x of tile y)
    ti = blockIdx.y;
    chunk = blockIdx.x;
    return ti < nt;
  }
  const int id = blockIdx.x + gridDim.x * blockIdx.y, x = id & 7, j = id >> 3;
  const int t0 = (int)(((long long)nt * x) >> 3), t1 = (int)(((long long)nt * (x + 1)) >> 3);  // this XCD's tiles
  if (j >= (t1 - t0) * nc) return false;
  const int grp = j / (4 * nc), first = t0 + 4 * grp, in_grp = min(4, t1 - first);  // (the run's last group may be short)
  const int r = j - grp * 4 * nc;
  chunk = r / in_grp;
  ti = first + r - chunk * in_grp;
  return true;
}

// The global loads of one K step, held in registers until the step before it has been computed.
// (native vector types: arrays of HIP's uint4, a struct, stay in scratch memory when they are passed around)
typedef uint32_t g2_u4 __attribute__((ext_vector_type(4)));
template <int QT> struct StepRegs {
  g2_u4 a[4];                        // 4 x 16 int8 activation values
  g2_u4 w[QT == QT_Q8_0 ? 4 : 2];    // packed weights
  uint32_t qh[2];                    // Q5_K: the words of fifth bits of the two 16-byte units above
  g2_u4 h;                           // Q4_K / Q5_K header of the thread's row (Q8_0: .x = two f16 scales)
  float sa[4];                       // scale of the block whose first half the thread stages (even chunks only)
};

template <int QT>
__device__ __forceinline__ void step_load(StepRegs<QT>& r, const Gemm2Lds& L, const uint8_t* __restrict__ raw, size_t rows_total,
                                 int nsb, size_t row_base, int n0, int N, const signed char* __restrict__ aq,
                                 const float* __restrict__ asc, int M, int K, int s, int hh) {
  const int t = threadIdx.x;
  const int e0 = s * 256 + 128 * hh;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int id = t + 256 * i, row = id >> 3, c = id & 7;
    const int m = max(L.rowmap[row], 0);
    r.a[i] = *(const g2_u4*)(aq + (size_t)m * K + e0 + 16 * c);
    r.sa[i] = asc[(size_t)(s * 8 + 4 * hh + (c >> 1)) * M + m];
  }
  if constexpr (QT == QT_Q4_K || QT == QT_Q5_K) {
    const PlanesQ4K pl = planes_q4k(rows_total, nsb);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const int n = min(n0 + row, N - 1);
      r.w[i] = *(const g2_u4*)(raw + pl.qs + ((row_base + n) * nsb + s) * 128 + 64 * hh + 16 * c);
      if constexpr (QT == QT_Q5_K) r.qh[i] = *(const uint32_t*)(raw + pl.qh + ((row_base + n) * nsb + s) * 32 + 16 * hh + 4 * c);
    }
    const int n = min(n0 + (t >> 1), N - 1);
    r.h = *(const g2_u4*)(raw + pl.hdr + ((row_base + n) * nsb + s) * 16);
  } else if constexpr (QT == QT_IQ4_XS) {
    const PlanesIQ4XS pl = planes_iq4xs(rows_total, nsb);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const int n = min(n0 + row, N - 1);
      r.w[i] = *(const g2_u4*)(raw + pl.qs + ((row_base + n) * nsb + s) * 128 + 64 * hh + 16 * c);
    }
    const int n = min(n0 + (t >> 1), N - 1);
    const uint2 h = *(const uint2*)(raw + pl.hdr + ((row_base + n) * nsb + s) * 8);
    r.h.x = h.x;
    r.h.y = h.y;
  } else if constexpr (qt_nib16(QT)) {
    const PlanesQ40 pl = planes_q40(rows_total, nsb);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const int n = min(n0 + row, N - 1);
      r.w[i] = *(const g2_u4*)(raw + pl.qs + ((row_base + n) * nsb + s) * 128 + 64 * hh + 16 * c);
    }
    const int n = min(n0 + (t >> 1), N - 1);
    // (the scales of blocks 4 hh + 2 (t & 1) and the next: two f16, or -- MXFP4 -- two bytes)
    if constexpr (QT == QT_MXFP4)
      r.h.x = *(const unsigned short*)(raw + pl.d + ((row_base + n) * nsb + s) * 8 + 4 * hh + 2 * (t & 1));
    else
      r.h.x = *(const uint32_t*)(raw + pl.d + (((row_base + n) * nsb + s) * 8 + 4 * hh + 2 * (t & 1)) * 2);
  } else {
    const PlanesQ80 pl = planes_q80(rows_total, nsb);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id = t + 256 * i, row = id >> 3, c = id & 7;
      const int n = min(n0 + row, N - 1);
      r.w[i] = *(const g2_u4*)(raw + pl.qs + ((row_base + n) * nsb + s) * 256 + 128 * hh + 16 * c);
    }
    const int n = min(n0 + (t >> 1), N - 1);
    r.h.x = *(const uint32_t*)(raw + pl.d + (((row_base + n) * nsb + s) * 8 + 4 * hh + 2 * (t & 1)) * 2);
  }
}

// Registers -> LDS: int8 values, decoded weights, the four scale vectors.  Rows past the tile carry zero scales.
template <int QT>
__device__ __forceinline__ void step_store(const StepRegs<QT>& r, Gemm2Lds& L, int hh) {
  constexpr bool Q45 = QT == QT_Q4_K || QT == QT_Q5_K;
  const int t = threadIdx.x;
  int ssum[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int id = t + 256 * i, row = id >> 3, c = id & 7;
    *(g2_u4*)&L.act[row][16 * c] = r.a[i];
    if constexpr (Q45) {
      int sh = dot4(r.a[i].x, 0x01010101u, 0);
      sh = dot4(r.a[i].y, 0x01010101u, sh);
      sh = dot4(r.a[i].z, 0x01010101u, sh);
      sh = dot4(r.a[i].w, 0x01010101u, sh);
      ssum[i] = sh + __shfl_xor(sh, 1, 64);  // the block's 32 values: this thread's 16 and its neighbour's
    }
    if ((c & 1) == 0) {  // rows past the tile carry zero scales
      const float sa = L.rowmap[row] >= 0 ? r.sa[i] : 0.0f;
      L.sa[c >> 1][row] = sa;
      if constexpr (Q45) L.u[c >> 1][row] = sa * (float)ssum[i];
    }
  }
  if constexpr (Q45) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const g2_u4 w = r.w[i];
      const int off = 64 * (c >> 1) + 16 * (c & 1);
      if constexpr (QT == QT_Q5_K) {
        const uint32_t H = r.qh[i];
        *(uint4*)&L.wq[row][off] = make_uint4(q5k_lo(w.x, H, 0), q5k_lo(w.y, H, 1), q5k_lo(w.z, H, 2), q5k_lo(w.w, H, 3));
        *(uint4*)&L.wq[row][off + 32] = make_uint4(q5k_hi(w.x, H, 0), q5k_hi(w.y, H, 1), q5k_hi(w.z, H, 2), q5k_hi(w.w, H, 3));
      } else {
        *(uint4*)&L.wq[row][off] = make_uint4(w.x & 0x0F0F0F0Fu, w.y & 0x0F0F0F0Fu, w.z & 0x0F0F0F0Fu, w.w & 0x0F0F0F0Fu);
        *(uint4*)&L.wq[row][off + 32] = make_uint4((w.x >> 4) & 0x0F0F0F0Fu, (w.y >> 4) & 0x0F0F0F0Fu,
                                                   (w.z >> 4) & 0x0F0F0F0Fu, (w.w >> 4) & 0x0F0F0F0Fu);
      }
    }
    {
      const int row = t >> 1, p = t & 1;
      const float d = f16_bits_to_f32(r.h.x), dmin = f16_bits_to_f32(r.h.x >> 16);
      int sc0, sc1, mn0, mn1;
      q4k_scales_pair(r.h.y, r.h.z, r.h.w, 2 * hh + p, sc0, sc1, mn0, mn1);
      L.ws[2 * p][row] = d * (float)sc0;
      L.ws[2 * p + 1][row] = d * (float)sc1;
      L.v[2 * p][row] = -(dmin * (float)mn0);
      L.v[2 * p + 1][row] = -(dmin * (float)mn1);
    }
  } else if constexpr (QT == QT_IQ4_XS) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {  // block 4 hh + c of the superblock: 16 bytes -> its 32 values
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const g2_u4 w = r.w[i];
      *(uint4*)&L.wq[row][32 * c] = make_uint4(iq4_lookup(w.x), iq4_lookup(w.y), iq4_lookup(w.z), iq4_lookup(w.w));
      *(uint4*)&L.wq[row][32 * c + 16] = make_uint4(iq4_lookup(w.x >> 4), iq4_lookup(w.y >> 4), iq4_lookup(w.z >> 4), iq4_lookup(w.w >> 4));
    }
    const int row = t >> 1, p = t & 1;
    const float d = f16_bits_to_f32(r.h.x);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int ib = 4 * hh + 2 * p + k;
      const int ls = (int)(((r.h.y >> (4 * ib)) & 0xFu) | ((((r.h.x >> 16) >> (2 * ib)) & 3u) << 4)) - 32;
      L.ws[2 * p + k][row] = d * (float)ls;
    }
  } else if constexpr (qt_nib16(QT)) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {  // block 4 hh + c of the superblock: 16 bytes -> its 32 values (nibble - 8, or the table's)
      const int id = t + 256 * i, row = id >> 2, c = id & 3;
      const g2_u4 w = r.w[i];
      *(uint4*)&L.wq[row][32 * c] = make_uint4(nib_vals<QT>(w.x), nib_vals<QT>(w.y), nib_vals<QT>(w.z), nib_vals<QT>(w.w));
      *(uint4*)&L.wq[row][32 * c + 16] = make_uint4(nib_vals<QT>(w.x >> 4), nib_vals<QT>(w.y >> 4), nib_vals<QT>(w.z >> 4), nib_vals<QT>(w.w >> 4));
    }
    const int row = t >> 1, p = t & 1;
    if constexpr (QT == QT_MXFP4) {
      L.ws[2 * p][row] = e8m0_half(r.h.x);
      L.ws[2 * p + 1][row] = e8m0_half(r.h.x >> 8);
    } else {
      L.ws[2 * p][row] = f16_bits_to_f32(r.h.x);
      L.ws[2 * p + 1][row] = f16_bits_to_f32(r.h.x >> 16);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id = t + 256 * i, row = id >> 3, c = id & 7;
      *(g2_u4*)&L.wq[row][16 * c] = r.w[i];
    }
    const int row = t >> 1, p = t & 1;
    L.ws[2 * p][row] = f16_bits_to_f32(r.h.x);
    L.ws[2 * p + 1][row] = f16_bits_to_f32(r.h.x >> 16);
  }
}

template <int QT, bool TILES>
__device__ __forceinline__ void gemm2_body(const uint8_t* __restrict__ raw, const signed char* __restrict__ aq,
                                  const float* __restrict__ asc, float* __restrict__ C, int M, int N, int K, int ldc,
                                  int c_off, int accumulate, int s_begin, int s_end, size_t rows_total, size_t row_base,
                                  int m0, int rows_valid, int n0, const int* __restrict__ rowmap, int use_map,
                                  const float* __restrict__ rowscale, int use_scale) {
  __shared__ Gemm2Lds L;
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // (a scalar: what follows from it alone is scalar arithmetic)
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

  StepRegs<QT> regs;
  const int steps = 2 * (s_end - s_begin);
  if (steps > 0) step_load<QT>(regs, L, raw, rows_total, nsb, row_base, n0, N, aq, asc, M, K, s_begin, 0);
  for (int st = 0; st < steps; ++st) {
    const int hh = st & 1;
    step_store<QT>(regs, L, hh);
    __syncthreads();
    if (st + 1 < steps)  // in flight during the products below
      step_load<QT>(regs, L, raw, rows_total, nsb, row_base, n0, N, aq, asc, M, K, s_begin + ((st + 1) >> 1), (st + 1) & 1);

    // 16 phases (block b, tile (ms, ns)).  Each phase first issues the matrix instructions of a later phase -- the
    // int8 product of the next tile and, every second phase, the outer product that makes the scale tiles of the next
    // token half -- and then spends its 32 ALU instructions on the current tile, so the matrix pipe works under the
    // ALU.  LDS operands are read one block ahead.
    v4i a16[2], w16[2];            // [ms], [ns]: reloaded for the next block as soon as their last product is issued
    float saop[2], wsop, uop[2], vop[2];
    v32f P[2];                     // scale tiles of (b, ms): [ms], both ns
    v16i I[2];                     // int sums of the current and the next tile
    auto ld_a = [&](int b, int ms) { a16[ms] = *(const v4i*)&L.act[wm * 64 + ms * 32 + l32][32 * b + 16 * g]; };
    auto ld_w = [&](int b, int ns) { w16[ns] = *(const v4i*)&L.wq[wn * 64 + ns * 32 + l32][32 * b + 16 * g]; };
    auto ld_sa = [&](int b, int ms) { saop[ms] = L.sa[b][wm * 64 + ms * 32 + l32]; };
    // lanes 0-31: columns of tile ns = 0, lanes 32-63: of ns = 1
    auto ld_ws = [&](int b) { wsop = L.ws[b][wn * 64 + lane]; };
    auto mfma_p = [&](int ms) {
      v32f zf;
#pragma unroll
      for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
      P[ms] = __builtin_amdgcn_mfma_f32_32x32x1f32(saop[ms], wsop, zf, 0, 0, 0);
    };
    auto mfma_i = [&](int ms, int ns, int slot) {
      v16i z;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] = 0;
      I[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[ms], w16[ns], z, 0, 0, 0);
    };
    ld_a(0, 0); ld_a(0, 1); ld_w(0, 0); ld_w(0, 1); ld_sa(0, 0); ld_sa(0, 1); ld_ws(0);
    mfma_p(0);
    mfma_i(0, 0, 0);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const bool more = b + 1 < 4;
      if constexpr (QT == QT_Q4_K || QT == QT_Q5_K) {
        if ((b & 1) == 0) {  // min term of blocks b and b + 1: lane half g supplies block b + g
#pragma unroll
          for (int ms = 0; ms < 2; ++ms) uop[ms] = L.u[b + g][wm * 64 + ms * 32 + l32];
#pragma unroll
          for (int ns = 0; ns < 2; ++ns) vop[ns] = L.v[b + g][wn * 64 + ns * 32 + l32];
        }
      }
#pragma unroll
      for (int tile = 0; tile < 4; ++tile) {
        const int ms = tile >> 1, ns = tile & 1, slot = tile & 1;
        // matrix instructions of later phases, and the LDS operands of the next block into registers just freed
        if (tile == 0) { mfma_i(0, 1, 1); }
        if (tile == 1) {
          mfma_p(1);
          mfma_i(1, 0, 0);
          if (more) { ld_a(b + 1, 0); ld_sa(b + 1, 0); }
        }
        if (tile == 2) {
          mfma_i(1, 1, 1);
          if (more) { ld_w(b + 1, 0); ld_ws(b + 1); }
        }
        if (tile == 3 && more) {
          mfma_p(0);
          mfma_i(0, 0, 0);
          ld_a(b + 1, 1); ld_w(b + 1, 1); ld_sa(b + 1, 1);
        }
        __builtin_amdgcn_sched_barrier(0);  // (keeps the matrix instructions above ahead of the ALU work below)
        // the current tile on the ALU
#pragma unroll
        for (int i = 0; i < 16; ++i)
          res[ms][ns][i] = __builtin_fmaf((float)I[slot][i], P[ms][16 * ns + i], res[ms][ns][i]);
        // the min term goes straight into the same accumulators on the matrix pipe; the ALU comes back to this tile
        // only after the other three
        if constexpr (QT == QT_Q4_K || QT == QT_Q5_K)
          if ((b & 1) == 0) res[ms][ns] = __builtin_amdgcn_mfma_f32_32x32x2f32(uop[ms], vop[ns], res[ms][ns], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
  }

  // ---- epilogue: lane = weight row n, accumulator i = token row 8 * (i / 4) + 4 * g + i % 4.  The slots' scales come
  // from LDS (read from global memory between the stores, each load would wait for the stores before it: one counter
  // orders both), and what the accumulate modes read of C is loaded for a whole tile before its first store.
  if (TILES && use_scale) {
    if (t < BM) L.sa[0][t] = t < rows_valid ? rowscale[m0 + t] : 0.0f;
    __syncthreads();
  }
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int ns = 0; ns < 2; ++ns) {
      const int n = n0 + wn * 64 + ns * 32 + l32;
      if (n >= N) continue;
      float cv[16];
      if (accumulate != 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int r = wm * 64 + ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          cv[i] = r < rows_valid ? C[(size_t)(m0 + r) * ldc + c_off + n] : 0.0f;
        }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = wm * 64 + ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
        if (r >= rows_valid) continue;
        float v = res[ms][ns][i];
        if (TILES && use_scale) v *= L.sa[0][r];
        if (accumulate == 1) {
          v += cv[i];
        } else if (accumulate == 2) {  // fused SwiGLU: C holds the gate projection, v the up projection
          v *= cv[i] / (1.0f + __expf(-cv[i]));
        }
        C[(size_t)(m0 + r) * ldc + c_off + n] = v;
      }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Q4_K, third form: the bulk operands go from global memory straight into LDS (global_load_lds_dwordx4: a wave moves
// 1 KB per instruction, lane l's 16 bytes land at base + 16 l, from whatever address lane l names), double-buffered,
// so the step after the current one streams in under the products with no registers and no ALU work; the weights
// stay packed in LDS (64 bytes per row and step) and are split into their two nibble blocks when a lane reads its
// operand.  Rows are not padded: the 16-byte chunk c of row r sits at chunk c ^ f(r), which the loading lane realises
// by choosing its source address, and which makes the 128-bit operand reads conflict-free.  Only the four scale vectors
// of a step pass through registers (they need arithmetic); S, the block sums of the activations, come from absum.
// One barrier per step.
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
__device__ inline v8bf as_bf16x8(v4u v) { return __builtin_bit_cast(v8bf, v); }
#define G3_STAGE 32768
#define G3_WQ 16384
#define G3_SA 24576
#define G3_U (G3_SA + 2048)
#define G3_WS (G3_SA + 4096)
#define G3_V (G3_SA + 6144)

// A result leaves for good: non-temporal stores keep the output (570 MB for 8192 tokens x 17408 rows, more than every
// cache) from displacing the operands that the neighbouring tiles still read (8192 tokens: 707 -> 717 TOP/s).  (Not for
// the expert tiles' y rows, which moe_combine reads right back: 56 -> 62 us there.)
__device__ inline void st_stream(float* p, float v) { __builtin_nontemporal_store(v, p); }

// (the 4-byte form: lane l's word lands at base + 4 l -- a gather of one value per lane)
__device__ inline void g3_dma4(const void* src, uint8_t* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 4, 0, 0);
}
__device__ inline void g3_dma16(const void* src, uint8_t* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

struct G3ScaleRegs {
  float sa[2];
  short bs[4];
  uint4 h;
};

// QT = Q5_K: the same with the fifth bits of a step's 128 values per row (16 bytes of the qh plane) brought into LDS by
// one more DMA instruction of the first two waves, and merged into the nibbles when a lane reads its operand.
// AU: the token side's two scale vectors come ready-made and go into LDS by DMA like the int8 rows -- asc itself and
// au[K / 32][M] = sa * S (act_usum in ops.hip makes it once per matmul) -- one more DMA instruction a wave and step in
// the place of six loads, the products and four LDS stores per thread; M must be a multiple of 4, the tile's first
// row of 128, and 512 bytes past the end of both arrays readable (rows past the chunk's last take what lies there:
// their results are not stored).
// PRE = 2: the row side's vectors too -- wsv = ws[K / 32][N] (d * sc) followed by v[K / 32][N] (-(dmin * mn)), made by
// q4k_wscales in front of a matmul of many tokens -- N a multiple of 4, 512 readable bytes past each: no scale
// arithmetic, no loads into registers and no LDS stores are left in the loop.
// PRE = 3 (Q4_K): the min term on the bf16 matrix instruction, which runs beside the vector ALU's work where the f32
// one does not (measured in this kernel: without the min term a launch takes 13 % less, with it on the bf16
// instruction 8 % less).  A float x is x1 + x2 + x3 exactly, three bf16 pieces by truncation; of the nine products of
// two such splits the eight without x3 y3 carry everything above 2^-32 of the product and fill the eight k-slots a
// lane half has in v_mfma_f32_32x32x16_bf16 (bf16 products are exact in f32, the sum is f32).  The pieces come
// ready-made: au[K / 32][M] entries (u1 | u2 << 16, u3 | u3 << 16), and behind ws in wsv v[K / 32][N] entries
// (v1 v1, v2 v2, v3 v3, v1 v2); a lane's token-side operand is the words (x, x, x, y) of its entry, its row-side
// operand the entry as it lies.  M even, 1 KB and 2 KB past the arrays' ends readable.  A stage is 40 KB.
// WM: the work-group's waves along the token rows, two rows of waves each way: 2 = 128 tokens x 128 rows in 4 waves, 4
// (PRE = 3 only) = 256 tokens x 128 rows in 8 waves of 64 x 64 -- one work-group a compute unit instead of two, the
// step's weight rows and row-side scale vectors brought into LDS once for 256 tokens instead of once for each 128.
template <bool TILES, int QT = QT_Q4_K, int PRE = 0, int WM = 2>  // (only the dense form is instantiated: over expert tiles,
                                                                 //  with their short K, the register-staged body measured faster)
__device__ __forceinline__ void gemm3_body(const uint8_t* __restrict__ raw, const signed char* __restrict__ aq,
                                  const float* __restrict__ asc, const short* __restrict__ absum, float* __restrict__ C,
                                  int M, int N, int K, int ldc, int c_off, int accumulate, int s_begin, int s_end,
                                  size_t rows_total, size_t row_base, int m0, int rows_valid, int n0,
                                  const int* __restrict__ rowmap, int use_map, const float* __restrict__ rowscale,
                                  int use_scale, const float* __restrict__ au = nullptr,
                                  const float* __restrict__ wsv = nullptr) {
  constexpr bool AU = PRE >= 1, WS = PRE >= 2;
  static_assert(!(AU && TILES), "the ready-made scale vectors are rows of the dense chunk");
  constexpr bool Q5 = QT == QT_Q5_K;
  constexpr bool BF = PRE >= 3;
  static_assert(!(BF && Q5), "the bf16 min-term form is built for Q4_K");
  // PRE = 4: the activations' scales are per 256 (the chunk's asc holds each eight times): a superblock's block sums
  // are added up as integers, sc * I per block in a 24-bit multiply-add, and meet the f32 scales once per superblock
  constexpr bool A256 = PRE == 4;
  static_assert(WM == 2 || (WM == 4 && PRE == 3), "the 256-token tile is built for the -DAU=3 form");
  constexpr int BMT = 64 * WM;        // token rows of the tile
  constexpr int NWI = 4 / WM;         // weight-row DMA instructions a wave and step (16 rows each)
  constexpr int oWQ = BMT * 128;      // the packed weight rows, behind the int8 token rows
  // the scale vectors of a stage: f32 per block and token / row (2 KB each), or, BF: sa, ws as before, then the min
  // term's operands, 8 bytes per block and token (4 KB) and 16 per block and row (8 KB): a stage of 40 KB
  constexpr int oSA = oWQ + 8192, oWS = BF ? oSA + 16 * BMT : G3_WS, oU = BF ? oWS + 2048 : G3_U, oV = BF ? oU + 32 * BMT : G3_V;
  constexpr int STAGE = BF ? oV + 8192 : Q5 ? G3_STAGE + 2048 : G3_STAGE, QH = G3_STAGE;  // (Q5_K: the fifth bits behind the scale vectors)
  static_assert(WM != 2 || (oWQ == G3_WQ && oSA == G3_SA && (!BF || STAGE == G3_SA + 16384)), "the 128-token layout");
  __shared__ alignas(16) uint8_t lds[2 * STAGE];
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // (a scalar: the DMA destinations and bases that follow from it are scalar arithmetic)
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  const PlanesQ4K pl = planes_q4k(rows_total, nsb);
  auto token_row = [&](int r) {  // global token row of tile row r; rows past the tile read the tile's first row
    const int rr = r < rows_valid ? r : 0;
    return (TILES && use_map) ? rowmap[m0 + rr] : m0 + rr;
  };

  // ---- what this lane fetches each step.  Activations: 4 instructions a wave, 8 rows each; row R = (4 wave + i) 8 +
  // lane / 8 lands at chunk lane % 8, so the lane names source chunk (lane % 8) ^ (R % 8).  Weights: 2 instructions a
  // wave, 16 rows each; row R = (2 wave + i) 16 + lane / 4, source chunk (lane % 4) ^ ((R / 2) % 4).
  // (per-lane parts as 32-bit byte offsets from bases that are the same for the whole wave and advance with the step)
  uint32_t aoff[4], woff[NWI];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int R = (wave * 4 + i) * 8 + (lane >> 3);
    aoff[i] = (uint32_t)token_row(R) * (uint32_t)K + 16u * ((lane & 7) ^ (lane >> 3));
  }
#pragma unroll
  for (int i = 0; i < NWI; ++i) {
    const int R = (wave * NWI + i) * 16 + (lane >> 2);
    const int n = min(n0 + R, N - 1);
    woff[i] = (uint32_t)n * (uint32_t)nsb * 128u + 16u * ((lane & 3) ^ ((lane >> 3) & 3));
  }
  const signed char* abase = aq + (size_t)s_begin * 256;
  const uint8_t* wbase = raw + pl.qs + (row_base * nsb + s_begin) * 128;
  // Q5_K: row R = 64 wave + lane (waves 0 and 1) brings the 16 bytes of its step's fifth bits to QH + 16 R
  const uint8_t* qbase = raw + pl.qh + (row_base * nsb + s_begin) * 32;
  uint32_t qoff = (uint32_t)min(n0 + (wave & 1) * 64 + lane, N - 1) * (uint32_t)nsb * 32u;
  // scales: thread t prepares token r_s = t % 128, blocks 2 (t / 128) + {0, 1} of the step, and weight row t / 2,
  // block pair t % 2
  const int r_s = t & 127, bp = t >> 7;
  const bool tok_valid = r_s < rows_valid;
  const uint32_t m_s = (uint32_t)token_row(r_s);
  const int n_s = min(n0 + (t >> 1), N - 1), p_s = t & 1;
  const uint32_t hoff = (uint32_t)n_s * (uint32_t)nsb * 16u;
  const uint8_t* hbase = raw + pl.hdr + (row_base * nsb + s_begin) * 16;
  // AU: waves 0 and 1 bring sa of blocks (0, 1) and (2, 3) of the step, waves 2 and 3 sa * S of the same: lane l the
  // four tokens 4 (l % 32) .. + 3 of block 2 (wave % 2) + l / 32
  const uint8_t* sbase = (const uint8_t*)(wave < 2 ? asc : au) + (size_t)s_begin * 8 * M * 4;
  uint32_t soff = ((uint32_t)(2 * (wave & 1) + (lane >> 5)) * (uint32_t)M + (uint32_t)m0 + 4u * (lane & 31)) * 4u;
  // WS: the same split for the row side: waves 0 and 1 d * sc, waves 2 and 3 -(dmin * mn), rows n0 + 4 (l % 32) .. + 3
  const uint8_t* rbase = (const uint8_t*)wsv + ((wave < 2 ? (size_t)0 : (size_t)(K >> 5) * N) + (size_t)s_begin * 8 * N) * 4;
  uint32_t roff = ((uint32_t)(2 * (wave & 1) + (lane >> 5)) * (uint32_t)N + (uint32_t)n0 + 4u * (lane & 31)) * 4u;
  // BF: waves 0 and 1 bring sa (asc), waves 2 and 3 d * sc (the f32 half of wsv), two blocks each as above; then wave w
  // the min term's operands of block w of the step: 128 token entries of 8 bytes (au: one instruction, lane l tokens
  // 2 l, 2 l + 1) and 128 row entries of 16 bytes (behind the f32 half of wsv: two instructions, lane l row 64 i + l)
  // (WM = 4: waves 0-3 bring sa of block w for the tile's 256 tokens, lane l the tokens 4 l .. + 3; waves 4 and 5 -- and 6
  //  and 7 once more, to the same place -- d * sc of blocks (0, 1) and (2, 3))
  const bool f_tok = WM == 4 ? wave < 4 : wave < 2;
  const uint8_t* fbase = f_tok ? (const uint8_t*)asc + (size_t)s_begin * 8 * M * 4 : (const uint8_t*)wsv + (size_t)s_begin * 8 * N * 4;
  const uint32_t fstep = 16u * (uint32_t)(f_tok ? M : N);  // (bytes of four blocks' f32 entries)
  uint32_t foff = WM == 4 ? (f_tok ? ((uint32_t)wave * (uint32_t)M + (uint32_t)m0 + 4u * lane) * 4u : roff) : (wave < 2 ? soff : roff);
  const int fdst = WM == 4 ? (f_tok ? oSA + wave * 1024 : oWS + (wave & 1) * 1024) : ((wave < 2 ? oSA : oWS) + (wave & 1) * 1024);
  // A256: wave 1 brings, in the place of sa of blocks 2 and 3, the superblock's d[n] (f32 [K / 256][N] behind the other
  // two parts of wsv), rows n0 + 4 (l % 32) .. + 3
  const uint8_t* dbase = (const uint8_t*)wsv + (size_t)(K >> 5) * N * 20 + (size_t)s_begin * N * 4;
  uint32_t doff = ((uint32_t)n0 + 4u * (lane & 31)) * 4u;
  // (the min term's operands: WM = 2, wave w brings block w -- 128 token entries in one instruction, 128 row entries in
  //  two; WM = 4, wave w brings block w / 2: the token entries 128 (w % 2) + 2 l, + 1 and the row entries 64 (w % 2) + l)
  const int mblk = WM == 4 ? wave >> 1 : wave;
  const uint8_t* ubase = (const uint8_t*)au + ((size_t)s_begin * 8 + mblk) * M * 8;
  uint32_t uoff = ((uint32_t)m0 + (WM == 4 ? 128u * (wave & 1) : 0u) + 2u * lane) * 8u;
  const int udst = WM == 4 ? oU + mblk * 2048 + (wave & 1) * 1024 : oU + wave * 1024;
  const uint8_t* vbase = (const uint8_t*)wsv + (size_t)(K >> 5) * N * 4 + ((size_t)s_begin * 8 + mblk) * N * 16;
  uint32_t voff = ((uint32_t)n0 + (WM == 4 ? 64u * (wave & 1) : 0u) + lane) * 16u;
  const int vdst = WM == 4 ? oV + mblk * 2048 + (wave & 1) * 1024 : oV + wave * 2048;

  auto dma_step = [&](int st, int stage) {  // st: half-superblock steps from s_begin
    uint8_t* base = lds + stage * STAGE;
    const signed char* ab = abase + (size_t)st * 128;
    const uint8_t* wb = wbase + (size_t)st * 64;
    // (the offsets pass through an empty asm so that the 64-bit addresses are formed here, each step, and not kept in
    //  twelve registers over the whole loop)
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(aoff[i]));
#pragma unroll
    for (int i = 0; i < 2; ++i) asm volatile("" : "+v"(woff[i]));
#pragma unroll
    for (int i = 0; i < 4; ++i) g3_dma16(ab + aoff[i], base + (wave * 4 + i) * 1024);
#pragma unroll
    for (int i = 0; i < 2; ++i) g3_dma16(wb + woff[i], base + G3_WQ + (wave * 2 + i) * 1024);
    if constexpr (Q5) {
      asm volatile("" : "+v"(qoff));
      if (wave < 2) g3_dma16(qbase + (size_t)st * 16 + qoff, base + QH + wave * 1024);
    }
  };
  // the same instructions one at a time (piece 0..7; Q5_K: 8 as well), for the forms that issue them between the
  // products instead of all at the head of the step: the memory pipe takes a wave's instruction every ~16 cycles and
  // eight waves of the compute unit ask at once, so a wave that issues all of its loads first stands in that queue
  // before its first product
  auto dma_piece = [&](int st, int stage, int piece) {
    uint8_t* base = lds + stage * STAGE;
    if (piece < 4) {
      asm volatile("" : "+v"(aoff[piece]));
      g3_dma16(abase + (size_t)st * 128 + aoff[piece], base + (wave * 4 + piece) * 1024);
    } else if (piece < 4 + NWI) {
      asm volatile("" : "+v"(woff[piece - 4]));
      g3_dma16(wbase + (size_t)st * 64 + woff[piece - 4], base + oWQ + (wave * NWI + piece - 4) * 1024);
    } else if constexpr (BF) {
      if (piece == 4 + NWI) {
        if (A256 && wave == 1) {
          asm volatile("" : "+v"(doff));
          g3_dma16(dbase + (size_t)(st >> 1) * N * 4 + doff, base + oSA + 1024);
        } else {
          asm volatile("" : "+v"(foff));
          g3_dma16(fbase + (size_t)st * fstep + foff, base + fdst);
        }
      } else if (piece == 5 + NWI) {
        asm volatile("" : "+v"(uoff));
        g3_dma16(ubase + (size_t)st * 4 * M * 8 + uoff, base + udst);
      } else if (piece < 6 + 2 * NWI) {  // (WM = 2: two instructions for the wave's 128 row entries; WM = 4: one for its 64)
        asm volatile("" : "+v"(voff));
        g3_dma16(vbase + (size_t)st * 4 * N * 16 + voff + (piece - 6 - NWI) * 1024, base + vdst + (piece - 6 - NWI) * 1024);
      }
    } else if (piece == 6) {
      asm volatile("" : "+v"(soff));
      g3_dma16(sbase + (size_t)st * 4 * M * 4 + soff, base + (wave < 2 ? oSA : oU) + (wave & 1) * 1024);
    } else if (piece == 7) {
      if constexpr (WS) {
        asm volatile("" : "+v"(roff));
        g3_dma16(rbase + (size_t)st * 4 * N * 4 + roff, base + (wave < 2 ? oWS : oV) + (wave & 1) * 1024);
      }
    } else if constexpr (Q5) {  // (no branch: waves 2 and 3 bring what waves 0 and 1 bring, to the same place)
      asm volatile("" : "+v"(qoff));
      g3_dma16(qbase + (size_t)st * 16 + qoff, base + QH + (wave & 1) * 1024);
    }
  };
  // (loads only: anything computed from them here would make the wave wait for the whole step's traffic)
  auto load_scales = [&](G3ScaleRegs& r, int st) {
    if constexpr (!AU) {
      const float* ap = asc + (size_t)(s_begin * 8 + st * 4 + 2 * bp) * M;
      const short* bp2 = absum + (size_t)(s_begin * 16 + st * 8 + 4 * bp) * M;
      r.sa[0] = ap[m_s];
      r.sa[1] = (ap + M)[m_s];
      r.bs[0] = bp2[m_s];
      r.bs[1] = (bp2 + M)[m_s];
      r.bs[2] = (bp2 + 2 * (size_t)M)[m_s];
      r.bs[3] = (bp2 + 3 * (size_t)M)[m_s];
    }
    if constexpr (!WS) r.h = *(const uint4*)(hbase + (size_t)(st >> 1) * 16 + hoff);
  };
  auto store_scales = [&](const G3ScaleRegs& r, int st, int stage) {
    uint8_t* base = lds + stage * STAGE;
    if constexpr (WS) return;
    if constexpr (!AU) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const float sa = tok_valid ? r.sa[q] : 0.0f;
        ((float*)(base + oSA))[(2 * bp + q) * 128 + r_s] = sa;
        ((float*)(base + oU))[(2 * bp + q) * 128 + r_s] = sa * (float)((int)r.bs[2 * q] + (int)r.bs[2 * q + 1]);
      }
    }
    const float d = f16_bits_to_f32(r.h.x), dmin = f16_bits_to_f32(r.h.x >> 16);
    int sc0, sc1, mn0, mn1;
    q4k_scales_pair(r.h.y, r.h.z, r.h.w, 2 * (st & 1) + p_s, sc0, sc1, mn0, mn1);
    const int row = t >> 1;
    ((float*)(base + oWS))[(2 * p_s) * 128 + row] = d * (float)sc0;
    ((float*)(base + oWS))[(2 * p_s + 1) * 128 + row] = d * (float)sc1;
    ((float*)(base + oV))[(2 * p_s) * 128 + row] = -(dmin * (float)mn0);
    ((float*)(base + oV))[(2 * p_s + 1) * 128 + row] = -(dmin * (float)mn1);
  };

  // ---- operand addresses of this lane (bytes from a stage's start)
  int oa[4], ow[2];
#pragma unroll
  for (int b = 0; b < 4; ++b) oa[b] = (wm * 64 + l32) * 128 + (((2 * b + g) ^ (l32 & 7)) * 16);
#pragma unroll
  for (int jj = 0; jj < 2; ++jj) ow[jj] = oWQ + (wn * 64 + l32) * 64 + (((2 * jj + g) ^ ((l32 >> 1) & 3)) * 16);

  v16f res[2][2];
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int ns = 0; ns < 2; ++ns)
#pragma unroll
      for (int i = 0; i < 16; ++i) res[ms][ns][i] = 0.0f;

  constexpr int NPIECE = BF ? 6 + 2 * NWI : 10;  // the DMA instructions of a wave and step (the forms below BF: up to 9, Q5_K's included)
  const int steps = 2 * (s_end - s_begin);
  G3ScaleRegs sr;
  if (steps > 0) {
    if constexpr (AU) {
#pragma unroll
      for (int p = 0; p < NPIECE; ++p) dma_piece(0, 0, p);
    } else {
      dma_step(0, 0);
    }
    load_scales(sr, 0);
    store_scales(sr, 0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the stage has landed
  }
  __syncthreads();

  for (int st = 0; st < steps; ++st) {
    const uint8_t* Sb = lds + (st & 1) * STAGE;
    const bool next = st + 1 < steps;
    if (next) {  // the other stage is free: every wave has passed the barrier that ended the step reading it
      if constexpr (!AU) dma_step(st + 1, (st + 1) & 1);  // (AU: one piece per product phase, below)
      load_scales(sr, st + 1);
    }

    v4i a16[2], w16[2], wraw[2];
    uint32_t h5[2];  // Q5_K: the fifth bits of the unit in wraw
    float saop[2], wsop, uop[2], vop[2];
    v4u uopb[2], vopb[2];  // BF: the min term's bf16 operands
    v32f P[2];
    v16i I[2];
    auto ld_a = [&](int b, int ms) { a16[ms] = *(const v4i*)(Sb + oa[b] + ms * 32 * 128); };
    auto ld_wraw = [&](int jj, int ns) {
      wraw[ns] = *(const v4i*)(Sb + ow[jj] + ns * 32 * 64);
      if constexpr (Q5) h5[ns] = *(const uint32_t*)(Sb + QH + (wn * 64 + ns * 32 + l32) * 16 + 4 * (2 * jj + g));
    };
    auto dec_w = [&](int b, int ns) {  // block b of the step: low nibbles of its pair's bytes if even, high if odd
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (Q5)
          w16[ns][i] = (b & 1) ? (int)q5k_hi((uint32_t)wraw[ns][i], h5[ns], i) : (int)q5k_lo((uint32_t)wraw[ns][i], h5[ns], i);
        else
          w16[ns][i] = (b & 1) ? (int)(((uint32_t)wraw[ns][i] >> 4) & 0x0F0F0F0Fu) : (int)((uint32_t)wraw[ns][i] & 0x0F0F0F0Fu);
      }
    };
    auto ld_sa = [&](int b, int ms) { saop[ms] = ((const float*)(Sb + oSA))[b * BMT + wm * 64 + ms * 32 + l32]; };
    auto ld_ws = [&](int b) { wsop = ((const float*)(Sb + oWS))[b * 128 + wn * 64 + lane]; };
    auto mfma_p = [&](int ms) {
      v32f zf;
#pragma unroll
      for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
      P[ms] = __builtin_amdgcn_mfma_f32_32x32x1f32(saop[ms], wsop, zf, 0, 0, 0);
    };
    auto mfma_i = [&](int ms, int ns, int slot) {
      v16i z;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] = 0;
      I[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[ms], w16[ns], z, 0, 0, 0);
    };
    if constexpr (A256) {
      // One row tile (ns) at a time, its two token tiles' integer sums J over the step's four blocks in registers: a
      // block's weights are decoded once, its sum is sc * I in a 24-bit multiply-add (|I| <= 32 x 127 x 15, sc <= 63), and
      // the four blocks' total meets the f32 scales once, as (sa[t] d[n]) tiles from the outer-product instruction.
      // The next step's loads go out one per product.  Then the min term as in the -DAU=3 form.
      const float dop = ((const float*)(Sb + oSA + 1024))[wn * 64 + lane];
      int piece = 0;
#pragma unroll
      for (int ns = 0; ns < 2; ++ns) {
        v16i Jt[2];
#pragma unroll
        for (int ms = 0; ms < 2; ++ms)
#pragma unroll
          for (int i = 0; i < 16; ++i) Jt[ms][i] = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          if ((b & 1) == 0) ld_wraw(b >> 1, ns);
          dec_w(b, ns);
          const int scn = ((const int*)(Sb + oWS))[b * 128 + wn * 64 + ns * 32 + l32];
#pragma unroll
          for (int ms = 0; ms < 2; ++ms) {
            ld_a(b, ms);
            mfma_i(ms, ns, ms);
            if (piece < 10) dma_piece(next ? st + 1 : st, (st + 1) & 1, piece);
            ++piece;
          }
#pragma unroll
          for (int ms = 0; ms < 2; ++ms)
#pragma unroll
            for (int i = 0; i < 16; ++i) Jt[ms][i] = __mul24(I[ms][i], scn) + Jt[ms][i];
        }
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
          const float sa256 = ((const float*)(Sb + oSA))[wm * 64 + ms * 32 + l32];
          v32f zf;
#pragma unroll
          for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
          const v32f Pd = __builtin_amdgcn_mfma_f32_32x32x1f32(sa256, dop, zf, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 16; ++i) res[ms][ns][i] = __builtin_fmaf((float)Jt[ms][i], Pd[16 * ns + i], res[ms][ns][i]);
        }
      }
#pragma unroll
      for (int b = 0; b < 4; b += 2) {
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
          const uint2 e = ((const uint2*)(Sb + oU))[(b + g) * 128 + wm * 64 + ms * 32 + l32];
          uopb[ms] = v4u{e.x, e.x, e.x, e.y};
        }
#pragma unroll
        for (int ns = 0; ns < 2; ++ns) vopb[ns] = *(const v4u*)(Sb + oV + ((b + g) * 128 + wn * 64 + ns * 32 + l32) * 16);
#pragma unroll
        for (int ms = 0; ms < 2; ++ms)
#pragma unroll
          for (int ns = 0; ns < 2; ++ns)
            res[ms][ns] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(uopb[ms]), as_bf16x8(vopb[ns]), res[ms][ns], 0, 0, 0);
      }
    } else {
    ld_wraw(0, 0); ld_wraw(0, 1); ld_a(0, 0); ld_a(0, 1); ld_sa(0, 0); ld_sa(0, 1); ld_ws(0);
    dec_w(0, 0); dec_w(0, 1);
    mfma_p(0);
    mfma_i(0, 0, 0);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const bool more = b + 1 < 4;
      if ((b & 1) == 0) {  // min term of blocks b and b + 1: lane half g supplies block b + g
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
          if constexpr (BF) {  // slots (u1 u2 | u1 u2 | u1 u2 | u3 u3) against the row side's (v1 v1 | v2 v2 | v3 v3 | v1 v2)
            const uint2 e = ((const uint2*)(Sb + oU))[(b + g) * BMT + wm * 64 + ms * 32 + l32];
            uopb[ms] = v4u{e.x, e.x, e.x, e.y};
          } else {
            uop[ms] = ((const float*)(Sb + oU))[(b + g) * 128 + wm * 64 + ms * 32 + l32];
          }
        }
#pragma unroll
        for (int ns = 0; ns < 2; ++ns) {
          if constexpr (BF)
            vopb[ns] = *(const v4u*)(Sb + oV + ((b + g) * 128 + wn * 64 + ns * 32 + l32) * 16);
          else
            vop[ns] = ((const float*)(Sb + oV))[(b + g) * 128 + wn * 64 + ns * 32 + l32];
        }
      }
#pragma unroll
      for (int tile = 0; tile < 4; ++tile) {
        const int ms = tile >> 1, ns = tile & 1, slot = tile & 1;
        if (tile == 0) {
          mfma_i(0, 1, 1);
          if (b == 1) { ld_wraw(1, 0); ld_wraw(1, 1); }  // (both nibble blocks of the first pair are in w16 by now)
        }
        if (tile == 1) {
          mfma_p(1);
          mfma_i(1, 0, 0);
          if (more) { ld_a(b + 1, 0); ld_sa(b + 1, 0); }
        }
        if (tile == 2) {
          mfma_i(1, 1, 1);
          if (more) { dec_w(b + 1, 0); ld_ws(b + 1); }
        }
        if (tile == 3 && more) {
          dec_w(b + 1, 1);
          mfma_p(0);
          mfma_i(0, 0, 0);
          ld_a(b + 1, 1); ld_sa(b + 1, 1);
        }
        if constexpr (AU) {  // the next step's loads, one instruction per phase over the first nine (no branch: the
                             //  last step brings its own stage once more, into the stage nobody reads)
          if (4 * b + tile < (BF ? NPIECE : 9)) dma_piece(next ? st + 1 : st, (st + 1) & 1, 4 * b + tile);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i)
          res[ms][ns][i] = __builtin_fmaf((float)I[slot][i], P[ms][16 * ns + i], res[ms][ns][i]);
        if ((b & 1) == 0) {
          if constexpr (BF)
            res[ms][ns] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(uopb[ms]), as_bf16x8(vopb[ns]), res[ms][ns], 0, 0, 0);
          else
            res[ms][ns] = __builtin_amdgcn_mfma_f32_32x32x2f32(uop[ms], vop[ns], res[ms][ns], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    }  // (!A256)
    if (next) {
      store_scales(sr, st + 1, (st + 1) & 1);
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();
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
        } else if (accumulate == 2) {
          const float gt = *cp;
          v *= gt / (1.0f + __expf(-gt));
        }
        st_stream(cp, v);
      }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Q6_K, dense.  Same machinery as the Q4_K kernel above (operands straight into double-buffered LDS, weights kept packed
// and rebuilt when a lane reads its operand, scale tile from an outer-product MFMA), shaped for the format's int8
// sub-scale per 16 values: a work-group computes 64 tokens x 128 weight rows, wave w all 64 tokens (two 32-row MFMA
// tiles) of rows [32 w, 32 w + 32), so every weight value is rebuilt by exactly one lane of the work-group.  A lane of
// the 32x32x32 product supplies the 16 values of sub-block g = lane / 32 of a block; two products with the other
// sub-block's lanes zeroed give the two sub-block sums I0, I1, and
//     res += (sa[m][b] * d[n] / 4) * (float)(sc0 * I0 + sc1 * I1)
// (four ALU instructions per product and block).  The weights enter the product as 4 (q - 32): the six bits of q with
// bit 5 flipped are q - 32 in six-bit two's complement, and moved to the top of a byte they are that number times 4.
#define G6_BM 64
#define G6_STAGE 23040
#define G6_QL 8192
#define G6_QH 16384
#define G6_SA 20480
#define G6_D 21504
#define G6_SC 22016

struct G6ScaleRegs {
  float sa;
  uint32_t sc;
  uint32_t d;
};

// Epilogue of the 64-slot bodies (a wave holds all 64 slots of its 32 weight rows: lane = row, accumulator i of tile ms
// = slot 32 ms + 8 (i / 4) + 4 g + i % 4) for a whole tile of 128 rows whose output rows are 16-byte aligned: the sums
// go through LDS (the stages are free: every wave is past the last step's barrier), slot r at 528 r bytes behind the
// slots' scales -- 16 bytes of padding keep the two lane halves, four slots apart, on different banks -- so that a
// thread writes 16 bytes and a wave two whole 512-byte rows of the tile: 8 store instructions a lane instead of 32,
// each over half as many lines.  What the accumulate modes read of C is loaded for all 8 before the first store, and
// the slots' scales come from LDS: loads between the stores would each wait for the stores before them (one counter
// orders both), 32 round trips to memory in a row.  false: not such a tile, nothing done (the caller's scalar path).
__device__ __forceinline__ bool store_tile64(uint8_t* lds, const v16f (&res)[2], float* __restrict__ C, int ldc, int c_off,
                                             int accumulate, int m0, int rows_valid, int n0, int N,
                                             const float* __restrict__ rowscale, int use_scale) {
  if (n0 + BN > N || ((ldc | c_off) & 3) != 0 || ((uintptr_t)C & 15) != 0) return false;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), l32 = lane & 31, g = lane >> 5;
  float* rs = (float*)lds;
  uint8_t* tl = lds + 256;
  if (use_scale && t < G6_BM) rs[t] = t < rows_valid ? rowscale[m0 + t] : 0.0f;
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      *(float*)(tl + (ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3)) * 528 + (wave * 32 + l32) * 4) = res[ms][i];
  const int c4 = t & 31, rr = t >> 5;
  float* cp = C + (size_t)(m0 + rr) * ldc + c_off + n0 + 4 * c4;
  float4 cv[8];
  if (accumulate != 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      cv[i] = rr + 8 * i < rows_valid ? *(const float4*)(cp + (size_t)8 * i * ldc) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = rr + 8 * i;
    if (r >= rows_valid) continue;
    float4 v = *(const float4*)(tl + r * 528 + c4 * 16);
    if (use_scale) {
      const float sc = rs[r];
      v.x *= sc; v.y *= sc; v.z *= sc; v.w *= sc;
    }
    if (accumulate == 1) {
      v.x += cv[i].x; v.y += cv[i].y; v.z += cv[i].z; v.w += cv[i].w;
    } else if (accumulate == 2) {  // fused SwiGLU: C holds the gate projection, v the up projection
      v.x *= cv[i].x / (1.0f + __expf(-cv[i].x));
      v.y *= cv[i].y / (1.0f + __expf(-cv[i].y));
      v.z *= cv[i].z / (1.0f + __expf(-cv[i].z));
      v.w *= cv[i].w / (1.0f + __expf(-cv[i].w));
    }
    *(float4*)(cp + (size_t)8 * i * ldc) = v;
  }
  return true;
}

// The gate/up tile's h = silu(gate) * up, stored as store_tile64 stores it, and quantized on the way out as the expert
// inputs' quantizer does (moe_quant_sums in moe.hip: per 32 values amax, q = rte(v * (127 / amax)), scale amax / 127,
// the sums of 16 -- the same helper, the same bits): the tile lies in LDS slot-major for the stores, a thread takes
// two half blocks of 16 values (neighbouring lanes the two halves of a block), writes their int8 values, and the
// scales and sums leave through LDS in rows of 64 slots.  hq [S][F], hsc [F/32][S], hbs [F/16][S].  Whole tiles of 128
// rows only (F a multiple of 128).
__device__ __forceinline__ void store_tile64_quant(uint8_t* lds, const v16f (&hv)[2], float* __restrict__ H, int F, int m0,
                                                   int rows_valid, int n0, int S, signed char* __restrict__ hq,
                                                   float* __restrict__ hsc, short* __restrict__ hbs,
                                                   float* __restrict__ hu = nullptr) {
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), l32 = lane & 31, g = lane >> 5;
  uint8_t* tl = lds + 256;
  float* lasc = (float*)(lds + 256 + 64 * 528);       // [4][64]
  short* lsum = (short*)(lds + 256 + 64 * 528 + 1024);  // [8][64]
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      *(float*)(tl + (ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3)) * 528 + (wave * 32 + l32) * 4) = hv[ms][i];
  __syncthreads();
  const int c4 = t & 31, rr = t >> 5;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = rr + 8 * i;
    if (r < rows_valid) *(float4*)(H + (size_t)(m0 + r) * F + n0 + 4 * c4) = *(const float4*)(tl + r * 528 + c4 * 16);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = t + 256 * i, hb = idx & 7, r = idx >> 3;
    float v[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 f = *(const float4*)(tl + r * 528 + hb * 64 + q * 16);
      v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
    }
    const float amax = block_amax(v, 1);
    uint4 pk;
    int sum;
    quant16(v, amax, pk, sum);
    if (r < rows_valid) *(uint4*)(hq + (size_t)(m0 + r) * F + n0 + hb * 16) = pk;
    if ((hb & 1) == 0) lasc[(hb >> 1) * 64 + r] = amax / 127.0f;
    lsum[hb * 64 + r] = (short)sum;
  }
  __syncthreads();
  {
    const int b = t >> 6, r = t & 63;
    if (r < rows_valid) hsc[((size_t)(n0 >> 5) + b) * S + m0 + r] = lasc[b * 64 + r];
    // (hu [F/32][S]: scale times the block's sum, what act_usum would make of hsc and hbs, for the down kernel's PRE form)
    if (hu && r < rows_valid)
      hu[((size_t)(n0 >> 5) + b) * S + m0 + r] = lasc[b * 64 + r] * (float)((int)lsum[2 * b * 64 + r] + (int)lsum[(2 * b + 1) * 64 + r]);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int hb = b + 4 * i;
      if (r < rows_valid) hbs[((size_t)(n0 >> 4) + hb) * S + m0 + r] = lsum[hb * 64 + r];
    }
  }
}

// TILES: one expert tile -- the planes hold rows_total rows, the expert's N rows start at row_base, slot r of the tile
// reads token row rowmap[m0 + r] (use_map) and its results are scaled by rowscale[m0 + r] (use_scale).
// HD != 0: planes written out from a type with one scale per 32 values (IQ3_S, IQ3_XXS), so a block's two int8 sub-scales
// are equal: one product per block over all 32 values instead of two over 16, and sc * I in the place of
// sc0 * I0 + sc1 * I1.  HD == 1: the planes moreover hold half the values (IQ3_XXS: its magnitudes, up to 62, are even
// and enter halved, and d / 4, which an f16 cannot always hold, becomes d with half the factor here).
template <bool TILES = false, int HD = 0>
__device__ __forceinline__ void gemm6_body(const uint8_t* __restrict__ raw, const signed char* __restrict__ aq,
                                  const float* __restrict__ asc, float* __restrict__ C, int M, int N, int K, int ldc,
                                  int c_off, int accumulate, int s_begin, int s_end, int m0, int rows_valid, int n0,
                                  size_t rows_total = 0, size_t row_base = 0, const int* __restrict__ rowmap = nullptr,
                                  int use_map = 0, const float* __restrict__ rowscale = nullptr, int use_scale = 0) {
  // (HD != 0: in the place of d and the sub-scale bytes, 1.5 KiB, the four blocks' f32 row scales d * sc: 2 KiB)
  constexpr int STAGE = HD != 0 ? G6_D + 2048 : G6_STAGE;
  __shared__ alignas(16) uint8_t lds[2 * STAGE];
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // (a scalar: what follows from it alone is scalar arithmetic)
  const int l32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  const PlanesQ6K pl = planes_q6k(TILES ? rows_total : (size_t)N, nsb);
  auto token_row = [&](int r) {  // rows past the tile read its first row
    const int rr = r < rows_valid ? r : 0;
    return (TILES && use_map) ? rowmap[m0 + rr] : m0 + rr;
  };

  // ---- what this lane fetches each step (a step = half a superblock = 128 values).  Activations: 2 instructions a
  // wave, 8 rows each, row R = (2 wave + i) 8 + lane / 8 at chunk lane % 8 <- source chunk (lane % 8) ^ (R % 8).  Low
  // nibbles: 2 instructions, 16 rows each, row R = (2 wave + i) 16 + lane / 4 <- source chunk (lane % 4) ^ ((R / 2) % 4).
  // High bits: 1 instruction, 32 rows, row R = 32 wave + lane / 2 <- source chunk (lane % 2) ^ ((R / 4) % 2).
  uint32_t aoff[2], loff[2], hoff;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int R = (wave * 2 + i) * 8 + (lane >> 3);
    aoff[i] = (uint32_t)token_row(R) * (uint32_t)K + 16u * ((lane & 7) ^ (lane >> 3));
    const int R2 = (wave * 2 + i) * 16 + (lane >> 2);
    loff[i] = (uint32_t)min(n0 + R2, N - 1) * (uint32_t)nsb * 128u + 16u * ((lane & 3) ^ ((lane >> 3) & 3));
  }
  hoff = (uint32_t)min(n0 + wave * 32 + (lane >> 1), N - 1) * (uint32_t)nsb * 64u + 16u * ((lane & 1) ^ ((lane >> 3) & 1));
  const signed char* abase = aq + (size_t)s_begin * 256;
  const uint8_t* lbase = raw + pl.ql + (row_base * nsb + s_begin) * 128;
  const uint8_t* hbase = raw + pl.qh + (row_base * nsb + s_begin) * 64;
  // scales: threads 0-63 prepare token t (the step's 4 activation scales: one per thread and block -> 4 threads a
  // token would do; here thread t takes token t % 64, block t / 64); every thread prepares weight row t / 2: the four
  // sub-scales 4 (t % 2) .. + 3 of the step, and (t % 2 == 0) the row's d.
  const int r_s = t & 63, b_s = wave;
  const bool tok_valid = r_s < rows_valid;
  const uint32_t m_s = (uint32_t)token_row(r_s);
  const int n_s = min(n0 + (t >> 1), N - 1), p_s = t & 1;

  auto dma_step = [&](int st, int stage) {
    uint8_t* base = lds + stage * STAGE;
    const signed char* ab = abase + (size_t)st * 128;
    const uint8_t* lb = lbase + (size_t)st * 64;
    const uint8_t* hb = hbase + (size_t)st * 32;
#pragma unroll
    for (int i = 0; i < 2; ++i) g3_dma16(ab + aoff[i], base + (wave * 2 + i) * 1024);
#pragma unroll
    for (int i = 0; i < 2; ++i) g3_dma16(lb + loff[i], base + G6_QL + (wave * 2 + i) * 1024);
    g3_dma16(hb + hoff, base + G6_QH + wave * 1024);
  };
  auto load_scales = [&](G6ScaleRegs& r, int st) {
    const int sb = s_begin + (st >> 1), hh = st & 1;
    r.sa = (asc + (size_t)(sb * 8 + hh * 4 + b_s) * M)[m_s];
    r.sc = *(const uint32_t*)(raw + pl.sc + ((row_base + n_s) * nsb + sb) * 16 + 8 * hh + 4 * p_s);
    r.d = *(const unsigned short*)(raw + pl.d + ((row_base + n_s) * nsb + sb) * 2);
  };
  auto store_scales = [&](const G6ScaleRegs& r, int stage) {
    uint8_t* base = lds + stage * STAGE;
    ((float*)(base + G6_SA))[b_s * 64 + r_s] = tok_valid ? r.sa : 0.0f;
    if constexpr (HD != 0) {
      // blocks 2 p_s and 2 p_s + 1 of the step: their scale (the first of the two equal sub-scale bytes) times d
      const float dq = (HD == 1 ? 0.125f : 0.25f) * f16_bits_to_f32(r.d);  // (the weights enter as 4 (q - 32))
      ((float*)(base + G6_D))[(2 * p_s) * 128 + (t >> 1)] = dq * (float)(int)(signed char)(r.sc & 0xFFu);
      ((float*)(base + G6_D))[(2 * p_s + 1) * 128 + (t >> 1)] = dq * (float)(int)(signed char)((r.sc >> 16) & 0xFFu);
    } else {
      ((uint32_t*)(base + G6_SC))[(t >> 1) * 2 + p_s] = r.sc;
      if (p_s == 0) ((float*)(base + G6_D))[t >> 1] = 0.25f * f16_bits_to_f32(r.d);  // (the weights enter as 4 (q - 32))
    }
  };

  // ---- operand addresses of this lane (bytes from a stage's start)
  int oa[4], ol[2], oh;
#pragma unroll
  for (int b = 0; b < 4; ++b) oa[b] = l32 * 128 + (((2 * b + g) ^ (l32 & 7)) * 16);
#pragma unroll
  for (int j = 0; j < 2; ++j) ol[j] = G6_QL + (wave * 32 + l32) * 64 + (((2 * j + g) ^ ((l32 >> 1) & 3)) * 16);
  oh = G6_QH + (wave * 32 + l32) * 32 + ((g ^ ((l32 >> 2) & 1)) * 16);
  const uint32_t keep0 = g == 0 ? 0xFFFFFFFFu : 0u, keep1 = ~keep0;

  v16f res[2];
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int i = 0; i < 16; ++i) res[ms][i] = 0.0f;

  const int steps = 2 * (s_end - s_begin);
  G6ScaleRegs sr;
  if (steps > 0) {
    dma_step(0, 0);
    load_scales(sr, 0);
    store_scales(sr, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the stage has landed
  }
  __syncthreads();

#pragma unroll 1
  for (int st = 0; st < steps; ++st) {
    const uint8_t* Sb = lds + (st & 1) * STAGE;
    const bool next = st + 1 < steps;
    if (next) {
      dma_step(st + 1, (st + 1) & 1);
      load_scales(sr, st + 1);
    }
    // raw weights of the lane's row for the whole step: low nibbles of blocks (0, 2) and (1, 3), high bits of all four
    const v4i ql0 = *(const v4i*)(Sb + ol[0]), ql1 = *(const v4i*)(Sb + ol[1]), qh = *(const v4i*)(Sb + oh);
    uint2 scw = {0u, 0u};
    float dop = 0.0f;
    if constexpr (HD == 0) {
      scw = *(const uint2*)(Sb + G6_SC + (wave * 32 + l32) * 8);
      dop = ((const float*)(Sb + G6_D))[wave * 32 + l32];
    }
    v4i a16[2][2], w0[2], w1[2];  // [buffer][ms]; [buffer]
    float saop[2], wsop[2];
    v32f P[2];
    v16i I0[2], I1[2];
    auto ld_a = [&](int b, int buf) {
      a16[buf][0] = *(const v4i*)(Sb + oa[b]);
      a16[buf][1] = *(const v4i*)(Sb + oa[b] + 32 * 128);
      saop[buf] = ((const float*)(Sb + G6_SA))[b * 64 + lane];
      wsop[buf] = HD != 0 ? ((const float*)(Sb + G6_D))[b * 128 + wave * 32 + l32] : dop;  // (HD: the block's row scale)
    };
    auto dec_w = [&](int b, int buf) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lw = (uint32_t)((b & 1) ? ql1[i] : ql0[i]), hw = (uint32_t)qh[i];
        const uint32_t nib = (b >> 1) ? (lw >> 2) & 0x3C3C3C3Cu : (lw << 2) & 0x3C3C3C3Cu;
        const uint32_t top = b == 3 ? hw & 0xC0C0C0C0u : (hw << (6 - 2 * b)) & 0xC0C0C0C0u;
        const uint32_t w = (nib | top) ^ 0x80808080u;
        if constexpr (HD != 0) {
          w0[buf][i] = (int)w;
        } else {
          w0[buf][i] = (int)(w & keep0);
          w1[buf][i] = (int)(w & keep1);
        }
      }
    };
    auto mfma_p = [&](int buf) {
      v32f zf;
#pragma unroll
      for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
      P[buf] = __builtin_amdgcn_mfma_f32_32x32x1f32(saop[buf], wsop[buf], zf, 0, 0, 0);
    };
    auto mfma_i = [&](int buf, int ms, int slot) {
      v16i z;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] = 0;
      I0[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[buf][ms], w0[buf], z, 0, 0, 0);
      if constexpr (HD == 0) I1[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[buf][ms], w1[buf], z, 0, 0, 0);
    };
    ld_a(0, 0);
    dec_w(0, 0);
    mfma_p(0);
    mfma_i(0, 0, 0);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int buf = b & 1;
      const bool more = b + 1 < 4;
      // int8 sub-scales of block b: bytes 2 b and 2 b + 1 of the step's eight
      const uint32_t scword = b < 2 ? scw.x : scw.y;
      const int sc0 = (int)(scword << (24 - 16 * (b & 1))) >> 24, sc1 = (int)(scword << (16 - 16 * (b & 1))) >> 24;
#pragma unroll
      for (int ms = 0; ms < 2; ++ms) {
        const int slot = ms;
        if (ms == 0) {
          mfma_i(buf, 1, 1);
          if (more) { ld_a(b + 1, buf ^ 1); dec_w(b + 1, buf ^ 1); }
        } else if (more) {
          mfma_p(buf ^ 1);
          mfma_i(buf ^ 1, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int j = HD != 0 ? I0[slot][i] : __mul24(sc0, I0[slot][i]) + __mul24(sc1, I1[slot][i]);
          res[ms][i] = __builtin_fmaf((float)j, P[buf][16 * ms + i], res[ms][i]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    asm volatile("" : "+v"(res[0]), "+v"(res[1]));  // (the sums are complete before the branches below)
    if (next) {
      store_scales(sr, (st + 1) & 1);
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();
  }

  // ---- epilogue: lane = weight row n, accumulator i = token row 8 * (i / 4) + 4 * g + i % 4
  if (store_tile64(lds, res, C, ldc, c_off, accumulate, m0, rows_valid, n0, N, rowscale, TILES && use_scale)) return;
  const int n = n0 + wave * 32 + l32;
  if (n < N) {
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
        if (r >= rows_valid) continue;
        float v = res[ms][i];
        if (TILES && use_scale) v *= rowscale[m0 + r];
        float* cp = C + (size_t)(m0 + r) * ldc + c_off + n;
        if (accumulate == 1) {
          v += *cp;
        } else if (accumulate == 2) {
          const float gt = *cp;
          v *= gt / (1.0f + __expf(-gt));
        }
        *cp = v;
      }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Q4_K over expert tiles, in the shape of the Q6_K kernel above: 64 slots x 128 weight rows per work-group (tiles of 64
// fill better than tiles of 128 when an expert has a few hundred slots), wave w all 64 slots of rows [32 w, 32 w + 32)
// (each packed weight is split into its nibbles by exactly one lane of the work-group), scale tile per block from one
// outer-product MFMA (lane halves = the two slot tiles), min term of a block pair from one v_mfma_f32_32x32x2_f32 per
// slot tile into the result accumulators, S from absum.  (For the dense matrix the 128 x 128 kernel above measured
// faster: half the traffic from L2 per product.)
#define G4_STAGE 22528
#define G4_WQ 8192
#define G4_SA 16384
#define G4_U 17408
#define G4_WS 18432
#define G4_V 20480

struct G4ScaleRegs {
  float sa;
  short bs[2];
  uint4 h;
};

// TWO = false: tiles of at most 32 slots; the second slot tile, whose scales would all be zero, is left out (half
// the matrix and vector instructions of a step).
// QT = Q5_K: as in the 128 x 128 body, a step's fifth bits (16 bytes a row) by one more DMA of the first two waves.
// PRE: the four scale vectors of a step come ready-made and go into LDS by DMA like the int8 rows, as in the dense
// kernel's -DAU=2 form: the token side from asc itself and au[K / 32][M] = sa * S (act_usum), a value per slot gathered
// by 4-byte DMA (a slot's token is wherever the routing put it); the row side from wsv = ws[K / 32][rows_total] (d * sc)
// followed by v[K / 32][rows_total] (-(dmin * mn)), made once per tensor when it is uploaded (q4k_wscales: 8 bytes per
// 32 weights).  The same expressions as the kernel's own preparation, so the same bits; what leaves the step loop is,
// per thread, four loads, the 6-bit unpack, eight conversions and products, six LDS stores and their wait.
template <bool TWO = true, int QT = QT_Q4_K, bool PRE = false>
__device__ __forceinline__ void gemm4_body(const uint8_t* __restrict__ raw, const signed char* __restrict__ aq,
                                  const float* __restrict__ asc, const short* __restrict__ absum, float* __restrict__ C,
                                  int M, int N, int K, int ldc, int c_off, int accumulate, int s_begin, int s_end,
                                  size_t rows_total, size_t row_base, int m0, int rows_valid, int n0,
                                  const int* __restrict__ rowmap, int use_map, const float* __restrict__ rowscale,
                                  int use_scale, const float* __restrict__ au = nullptr,
                                  const float* __restrict__ wsv = nullptr) {
  static_assert(!PRE || QT == QT_Q4_K, "the ready-made scale vectors are built for Q4_K");
  constexpr bool Q5 = QT == QT_Q5_K;
  constexpr int STAGE = Q5 ? G4_STAGE + 2048 : G4_STAGE, QH = G4_STAGE;
  __shared__ alignas(16) uint8_t lds[2 * STAGE];
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // (a scalar: what follows from it alone is scalar arithmetic)
  const int l32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  const PlanesQ4K pl = planes_q4k(rows_total, nsb);
  auto token_row = [&](int r) {  // the token row slot r reads; slots past the tile read its first
    const int rr = m0 + (r < rows_valid ? r : 0);
    return use_map ? rowmap[rr] : rr;
  };

  uint32_t aoff[2], woff[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int R = (wave * 2 + i) * 8 + (lane >> 3);
    aoff[i] = (uint32_t)token_row(R) * (uint32_t)K + 16u * ((lane & 7) ^ (lane >> 3));
    const int R2 = (wave * 2 + i) * 16 + (lane >> 2);
    woff[i] = (uint32_t)min(n0 + R2, N - 1) * (uint32_t)nsb * 128u + 16u * ((lane & 3) ^ ((lane >> 3) & 3));
  }
  const signed char* abase = aq + (size_t)s_begin * 256;
  const uint8_t* wbase = raw + pl.qs + (row_base * nsb + s_begin) * 128;
  const uint8_t* qbase = raw + pl.qh + (row_base * nsb + s_begin) * 32;  // Q5_K: row 64 wave + lane, waves 0 and 1
  uint32_t qoff = (uint32_t)min(n0 + (wave & 1) * 64 + lane, N - 1) * (uint32_t)nsb * 32u;
  // scales: thread t prepares token t % 64, block t / 64 of the step, and weight row t / 2, block pair t % 2
  const int r_s = t & 63, b_s = wave;
  const bool tok_valid = r_s < rows_valid;
  const uint32_t m_s = (uint32_t)token_row(r_s);
  const int n_s = min(n0 + (t >> 1), N - 1), p_s = t & 1;
  // PRE: wave w brings sa and sa * S of block w of the step for the 64 slots (lane l: slot l's token), and one of the
  // four row-side pieces of 1 KB: waves 0 and 1 d * sc of blocks (0, 1) and (2, 3), waves 2 and 3 -(dmin * mn) of the
  // same -- lane l the rows 4 (l % 32) .. + 3 of block 2 (w % 2) + l / 32.  (A layout of wsv with a step's vectors of a
  // row side by side -- one run of 4 KB a step instead of eight pieces of 512 bytes rows_total * 4 bytes apart -- was
  // built and measured the same: 0.705-0.72 ms a layer either way.)
  uint32_t toff = (uint32_t)token_row(lane) * 4u;
  const uint8_t* tbase = (const uint8_t*)asc + ((size_t)s_begin * 8 + wave) * M * 4;
  const uint8_t* ubase = (const uint8_t*)au + ((size_t)s_begin * 8 + wave) * M * 4;
  const uint8_t* rbase = (const uint8_t*)wsv + ((wave < 2 ? (size_t)0 : (size_t)(K >> 5) * rows_total) + (size_t)s_begin * 8 * rows_total) * 4;
  uint32_t roff = ((uint32_t)(2 * (wave & 1) + (lane >> 5)) * (uint32_t)rows_total + (uint32_t)row_base + (uint32_t)n0 + 4u * (lane & 31)) * 4u;

  auto dma_step = [&](int st, int stage) {
    uint8_t* base = lds + stage * STAGE;
    const signed char* ab = abase + (size_t)st * 128;
    const uint8_t* wb = wbase + (size_t)st * 64;
#pragma unroll
    for (int i = 0; i < 2; ++i) g3_dma16(ab + aoff[i], base + (wave * 2 + i) * 1024);
#pragma unroll
    for (int i = 0; i < 2; ++i) g3_dma16(wb + woff[i], base + G4_WQ + (wave * 2 + i) * 1024);
    if constexpr (Q5) {
      asm volatile("" : "+v"(qoff));
      if (wave < 2) g3_dma16(qbase + (size_t)st * 16 + qoff, base + QH + wave * 1024);
    }
    if constexpr (PRE) {
      asm volatile("" : "+v"(toff), "+v"(roff));
      g3_dma4(tbase + (size_t)st * 4 * M * 4 + toff, base + G4_SA + wave * 256);
      g3_dma4(ubase + (size_t)st * 4 * M * 4 + toff, base + G4_U + wave * 256);
      g3_dma16(rbase + (size_t)st * 4 * rows_total * 4 + roff, base + (wave < 2 ? G4_WS : G4_V) + (wave & 1) * 1024);
    }
  };
  // (loads only: anything computed from them here would make the wave wait for the whole step's traffic)
  auto load_scales = [&](G4ScaleRegs& r, int st) {
    if constexpr (PRE) return;
    const int blk = s_begin * 8 + st * 4 + b_s;
    r.sa = (asc + (size_t)blk * M)[m_s];
    r.bs[0] = (absum + (size_t)(2 * blk) * M)[m_s];
    r.bs[1] = (absum + (size_t)(2 * blk + 1) * M)[m_s];
    r.h = *(const uint4*)(raw + pl.hdr + ((row_base + n_s) * nsb + s_begin + (st >> 1)) * 16);
  };
  auto store_scales = [&](const G4ScaleRegs& r, int st, int stage) {
    if constexpr (PRE) return;
    uint8_t* base = lds + stage * STAGE;
    const float sa = tok_valid ? r.sa : 0.0f;
    ((float*)(base + G4_SA))[b_s * 64 + r_s] = sa;
    ((float*)(base + G4_U))[b_s * 64 + r_s] = sa * (float)((int)r.bs[0] + (int)r.bs[1]);
    const float d = f16_bits_to_f32(r.h.x), dmin = f16_bits_to_f32(r.h.x >> 16);
    int sc0, sc1, mn0, mn1;
    q4k_scales_pair(r.h.y, r.h.z, r.h.w, 2 * (st & 1) + p_s, sc0, sc1, mn0, mn1);
    const int row = t >> 1;
    ((float*)(base + G4_WS))[(2 * p_s) * 128 + row] = d * (float)sc0;
    ((float*)(base + G4_WS))[(2 * p_s + 1) * 128 + row] = d * (float)sc1;
    ((float*)(base + G4_V))[(2 * p_s) * 128 + row] = -(dmin * (float)mn0);
    ((float*)(base + G4_V))[(2 * p_s + 1) * 128 + row] = -(dmin * (float)mn1);
  };

  int oa[4], ow[2];
#pragma unroll
  for (int b = 0; b < 4; ++b) oa[b] = l32 * 128 + (((2 * b + g) ^ (l32 & 7)) * 16);
#pragma unroll
  for (int j = 0; j < 2; ++j) ow[j] = G4_WQ + (wave * 32 + l32) * 64 + (((2 * j + g) ^ ((l32 >> 1) & 3)) * 16);

  v16f res[2];
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int i = 0; i < 16; ++i) res[ms][i] = 0.0f;

  const int steps = 2 * (s_end - s_begin);
  G4ScaleRegs sr;
  if (steps > 0) {
    dma_step(0, 0);
    load_scales(sr, 0);
    store_scales(sr, 0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the stage has landed
  }
  __syncthreads();

#pragma unroll 1
  for (int st = 0; st < steps; ++st) {
    const uint8_t* Sb = lds + (st & 1) * STAGE;
    const bool next = st + 1 < steps;
    if (next) {
      dma_step(st + 1, (st + 1) & 1);
      load_scales(sr, st + 1);
    }
    // packed weights of the lane's row for the whole step: block pairs (0, 1) and (2, 3)
    const v4i wr0 = *(const v4i*)(Sb + ow[0]), wr1 = *(const v4i*)(Sb + ow[1]);
    uint32_t h50 = 0, h51 = 0;  // Q5_K: the fifth bits of the units in wr0, wr1
    if constexpr (Q5) {
      h50 = *(const uint32_t*)(Sb + QH + (wave * 32 + l32) * 16 + 4 * g);
      h51 = *(const uint32_t*)(Sb + QH + (wave * 32 + l32) * 16 + 4 * (2 + g));
    }
    v4i a16[2][2], w16[2];  // [buffer][ms]; [buffer]
    float saop[2], wsop[2], uop[2], vop;
    v32f P[2];
    v16i I[2];
    auto ld_a = [&](int b, int buf) {
      a16[buf][0] = *(const v4i*)(Sb + oa[b]);
      if constexpr (TWO) a16[buf][1] = *(const v4i*)(Sb + oa[b] + 32 * 128);
      saop[buf] = ((const float*)(Sb + G4_SA))[b * 64 + lane];
      wsop[buf] = ((const float*)(Sb + G4_WS))[b * 128 + wave * 32 + l32];
    };
    auto dec_w = [&](int b, int buf) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t x = (uint32_t)((b >> 1) ? wr1[i] : wr0[i]);
        if constexpr (Q5) {
          const uint32_t H = (b >> 1) ? h51 : h50;
          w16[buf][i] = (int)((b & 1) ? q5k_hi(x, H, i) : q5k_lo(x, H, i));
        } else {
          w16[buf][i] = (int)((b & 1) ? (x >> 4) & 0x0F0F0F0Fu : x & 0x0F0F0F0Fu);
        }
      }
    };
    auto mfma_p = [&](int buf) {
      v32f zf;
#pragma unroll
      for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
      P[buf] = __builtin_amdgcn_mfma_f32_32x32x1f32(saop[buf], wsop[buf], zf, 0, 0, 0);
    };
    auto mfma_i = [&](int buf, int ms, int slot) {
      v16i z;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] = 0;
      I[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[buf][ms], w16[buf], z, 0, 0, 0);
    };
    ld_a(0, 0);
    dec_w(0, 0);
    mfma_p(0);
    mfma_i(0, 0, 0);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int buf = b & 1;
      const bool more = b + 1 < 4;
      if ((b & 1) == 0) {  // min term of blocks b and b + 1: lane half g supplies block b + g
#pragma unroll
        for (int ms = 0; ms < (TWO ? 2 : 1); ++ms) uop[ms] = ((const float*)(Sb + G4_U))[(b + g) * 64 + ms * 32 + l32];
        vop = ((const float*)(Sb + G4_V))[(b + g) * 128 + wave * 32 + l32];
      }
      if constexpr (TWO) {
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
          const int slot = ms;
          if (ms == 0) {
            mfma_i(buf, 1, 1);
            if (more) { ld_a(b + 1, buf ^ 1); dec_w(b + 1, buf ^ 1); }
          } else if (more) {
            mfma_p(buf ^ 1);
            mfma_i(buf ^ 1, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = 0; i < 16; ++i) res[ms][i] = __builtin_fmaf((float)I[slot][i], P[buf][16 * ms + i], res[ms][i]);
          if ((b & 1) == 0) res[ms] = __builtin_amdgcn_mfma_f32_32x32x2f32(uop[ms], vop, res[ms], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        // one slot tile: the next block's matrix instructions go out, then this block's products (slots alternate)
        if (more) {
          ld_a(b + 1, buf ^ 1);
          dec_w(b + 1, buf ^ 1);
          mfma_p(buf ^ 1);
          mfma_i(buf ^ 1, 0, buf ^ 1);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i) res[0][i] = __builtin_fmaf((float)I[buf][i], P[buf][i], res[0][i]);
        if ((b & 1) == 0) res[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(uop[0], vop, res[0], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    asm volatile("" : "+v"(res[0]), "+v"(res[1]));  // (the sums are complete before the branches below)
    if (next) {
      store_scales(sr, st + 1, (st + 1) & 1);
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();
  }

  // ---- epilogue: lane = weight row n, accumulator i = token row 8 * (i / 4) + 4 * g + i % 4
  if constexpr (TWO) {
    if (store_tile64(lds, res, C, ldc, c_off, accumulate, m0, rows_valid, n0, N, rowscale, use_scale)) return;
  }
  const int n = n0 + wave * 32 + l32;
  if (n < N) {
#pragma unroll
    for (int ms = 0; ms < (TWO ? 2 : 1); ++ms)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
        if (r >= rows_valid) continue;
        float v = res[ms][i];
        if (use_scale) v *= rowscale[m0 + r];
        float* cp = C + (size_t)(m0 + r) * ldc + c_off + n;
        if (accumulate == 1) {
          v += *cp;
        } else if (accumulate == 2) {
          const float gt = *cp;
          v *= gt / (1.0f + __expf(-gt));
        }
        *cp = v;
      }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Q4_K gate and up projections of a mixture-of-experts layer in one pass (the reference's moe_gateup_q,
// zero/kernels/decode_moe.cl:92-94: h = silu(gate) * up straight from the two raw expert tensors).  The tile body above
// with two weight streams: the 64 slots' activations are staged once for both, a wave computes its 32 rows of gate and
// of up (16 products a step instead of 8, the same barrier and loads-issue cost), and the epilogue writes h once --
// against two launches, the second reading the first's output back.
#define GU_STAGE 34816
#define GU_WQ0 8192
#define GU_WQ1 16384
#define GU_SA 24576
#define GU_U 25600
#define GU_WS0 26624
#define GU_V0 28672
#define GU_WS1 30720
#define GU_V1 32768

struct GuScaleRegs {
  float sa;
  short bs[2];
  uint4 h;
};

// GU: the two streams are gate and up of an expert (rows n0.. of both tensors, h = silu(gate) * up); otherwise they are
// rows n0.. and n0 + 128.. of one matrix and each gets the plain epilogue (a 64 x 256 tile of a dense product).
template <bool GU, bool QUANT = false>
__device__ __forceinline__ void gemm4gu_body(const uint8_t* __restrict__ rg, const uint8_t* __restrict__ ru,
                                    const signed char* __restrict__ aq, const float* __restrict__ asc,
                                    const short* __restrict__ absum, float* __restrict__ H, int M, int N, int K,
                                    size_t rows_total, size_t row_base, int m0, int rows_valid, int n0,
                                    const int* __restrict__ rowmap, int ldc, int c_off, int accumulate, int S = 0,
                                    signed char* __restrict__ hq = nullptr, float* __restrict__ hsc = nullptr,
                                    short* __restrict__ hbs = nullptr) {
  __shared__ alignas(16) uint8_t lds[2 * GU_STAGE];
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  const PlanesQ4K pl = planes_q4k(rows_total, nsb);
  auto token_row = [&](int r) {  // slots past the tile read its first
    const int rr = m0 + (r < rows_valid ? r : 0);
    return GU ? rowmap[rr] : rr;
  };
  const int nx[2] = {n0, GU ? n0 : n0 + 128};  // first row of each stream
  const uint8_t* raws[2] = {rg, ru};

  uint32_t aoff[2], woff[2][2];  // woff[stream][instruction]
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int R = (wave * 2 + i) * 8 + (lane >> 3);
    aoff[i] = (uint32_t)token_row(R) * (uint32_t)K + 16u * ((lane & 7) ^ (lane >> 3));
    const int R2 = (wave * 2 + i) * 16 + (lane >> 2);
#pragma unroll
    for (int x = 0; x < 2; ++x)
      woff[x][i] = (uint32_t)min(nx[x] + R2, N - 1) * (uint32_t)nsb * 128u + 16u * ((lane & 3) ^ ((lane >> 3) & 3));
  }
  const size_t wrow0 = pl.qs + row_base * nsb * 128;
  // scales: thread t prepares token t % 64, block t / 64 of the step, and weight row t % 128 of gate (t < 128) or up
  const int r_s = t & 63, b_s = wave;
  const bool tok_valid = r_s < rows_valid;
  const uint32_t m_s = (uint32_t)token_row(r_s);
  const int row_s = t & 127, x_s = wave >> 1;
  const uint8_t* hsrc = (x_s ? ru : rg) + pl.hdr + (row_base + min(nx[x_s] + row_s, N - 1)) * nsb * 16;
  auto dma_step = [&](int st, int stage) {
    uint8_t* base = lds + stage * GU_STAGE;
    const signed char* ab = aq + (size_t)st * 128;
    // (the offsets pass through an empty asm so that the 64-bit addresses are formed here, each step, and not kept in
    //  twelve registers over the whole loop)
#pragma unroll
    for (int i = 0; i < 2; ++i) asm volatile("" : "+v"(aoff[i]), "+v"(woff[0][i]), "+v"(woff[1][i]));
#pragma unroll
    for (int i = 0; i < 2; ++i) g3_dma16(ab + aoff[i], base + (wave * 2 + i) * 1024);
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const uint8_t* wb = raws[x] + wrow0 + (size_t)st * 64;
#pragma unroll
      for (int i = 0; i < 2; ++i) g3_dma16(wb + woff[x][i], base + (x ? GU_WQ1 : GU_WQ0) + (wave * 2 + i) * 1024);
    }
  };
  auto load_scales = [&](GuScaleRegs& r, int st) {
    const int blk = st * 4 + b_s;
    r.sa = (asc + (size_t)blk * M)[m_s];
    r.bs[0] = (absum + (size_t)(2 * blk) * M)[m_s];
    r.bs[1] = (absum + (size_t)(2 * blk + 1) * M)[m_s];
    r.h = *(const uint4*)(hsrc + (size_t)(st >> 1) * 16);
  };
  auto store_scales = [&](const GuScaleRegs& r, int st, int stage) {
    uint8_t* base = lds + stage * GU_STAGE;
    const float sa = tok_valid ? r.sa : 0.0f;
    ((float*)(base + GU_SA))[b_s * 64 + r_s] = sa;
    ((float*)(base + GU_U))[b_s * 64 + r_s] = sa * (float)((int)r.bs[0] + (int)r.bs[1]);
    const float d = f16_bits_to_f32(r.h.x), dmin = f16_bits_to_f32(r.h.x >> 16);
    float* ws = (float*)(base + (x_s ? GU_WS1 : GU_WS0));
    float* vv = (float*)(base + (x_s ? GU_V1 : GU_V0));
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      int sc0, sc1, mn0, mn1;
      q4k_scales_pair(r.h.y, r.h.z, r.h.w, 2 * (st & 1) + p, sc0, sc1, mn0, mn1);
      ws[(2 * p) * 128 + row_s] = d * (float)sc0;
      ws[(2 * p + 1) * 128 + row_s] = d * (float)sc1;
      vv[(2 * p) * 128 + row_s] = -(dmin * (float)mn0);
      vv[(2 * p + 1) * 128 + row_s] = -(dmin * (float)mn1);
    }
  };

  int oa[4], ow[2];
#pragma unroll
  for (int b = 0; b < 4; ++b) oa[b] = l32 * 128 + (((2 * b + g) ^ (l32 & 7)) * 16);
#pragma unroll
  for (int j = 0; j < 2; ++j) ow[j] = (wave * 32 + l32) * 64 + (((2 * j + g) ^ ((l32 >> 1) & 3)) * 16);

  v16f res[2][2];  // [gate / up][slot tile]
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int i = 0; i < 16; ++i) res[x][ms][i] = 0.0f;

  const int steps = 2 * nsb;
  GuScaleRegs sr;
  dma_step(0, 0);
  load_scales(sr, 0);
  store_scales(sr, 0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the stage has landed
  __syncthreads();

#pragma unroll 1
  for (int st = 0; st < steps; ++st) {
    const uint8_t* Sb = lds + (st & 1) * GU_STAGE;
    const bool next = st + 1 < steps;
    if (next) {
      dma_step(st + 1, (st + 1) & 1);
      load_scales(sr, st + 1);
    }
    // packed weights of the lane's rows, [gate / up]: the block pair in use (the second pair of the step is read into
    // the same registers once both blocks of the first are split off)
    v4i wr[2];
    auto ld_wr = [&](int j, int x) { wr[x] = *(const v4i*)(Sb + (x ? GU_WQ1 : GU_WQ0) + ow[j]); };
    ld_wr(0, 0); ld_wr(0, 1);
    v4i a16[2], w16[2];  // [slot tile], [gate / up]: reloaded for the next block as soon as their last product is issued
    float saop, wsop[2], uop[2], vop[2];
    v32f P[2];  // scale tiles of the block: [gate / up], both slot tiles
    v16i I[2];
    auto ld_a = [&](int b, int ms) { a16[ms] = *(const v4i*)(Sb + oa[b] + ms * 32 * 128); };
    auto ld_sa = [&](int b) { saop = ((const float*)(Sb + GU_SA))[b * 64 + lane]; };
    auto ld_ws = [&](int b, int x) { wsop[x] = ((const float*)(Sb + (x ? GU_WS1 : GU_WS0)))[b * 128 + wave * 32 + l32]; };
    auto dec_w = [&](int b, int x) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t v = (uint32_t)wr[x][i];
        w16[x][i] = (int)((b & 1) ? (v >> 4) & 0x0F0F0F0Fu : v & 0x0F0F0F0Fu);
      }
    };
    auto mfma_p = [&](int x) {
      v32f zf;
#pragma unroll
      for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
      P[x] = __builtin_amdgcn_mfma_f32_32x32x1f32(saop, wsop[x], zf, 0, 0, 0);
    };
    auto mfma_i = [&](int x, int ms, int slot) {
      v16i z;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] = 0;
      I[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[ms], w16[x], z, 0, 0, 0);
    };
    ld_a(0, 0); ld_a(0, 1); ld_sa(0); ld_ws(0, 0); ld_ws(0, 1);
    dec_w(0, 0); dec_w(0, 1);
    mfma_p(0);
    mfma_i(0, 0, 0);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const bool more = b + 1 < 4;
      if ((b & 1) == 0) {  // min term of blocks b and b + 1: lane half g supplies block b + g
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) uop[ms] = ((const float*)(Sb + GU_U))[(b + g) * 64 + ms * 32 + l32];
#pragma unroll
        for (int x = 0; x < 2; ++x) vop[x] = ((const float*)(Sb + (x ? GU_V1 : GU_V0)))[(b + g) * 128 + wave * 32 + l32];
      }
      // four phases: (gate, tile 0), (gate, tile 1), (up, tile 0), (up, tile 1); each issues the next phase's product
#pragma unroll
      for (int ph = 0; ph < 4; ++ph) {
        const int x = ph >> 1, ms = ph & 1, slot = ph & 1;
        if (ph == 0) {
          mfma_i(0, 1, 1);                      // (gate, 1)
          if (more) {                           // gate's operand of the next block (this block's is issued twice by now)
            dec_w(b + 1, 0);
            if (b == 0) ld_wr(1, 0);
          }
        }
        if (ph == 1) {
          mfma_p(1);                            // up's scale tiles of this block
          mfma_i(1, 0, 0);                      // (up, 0)
          if (more) { ld_a(b + 1, 0); ld_sa(b + 1); ld_ws(b + 1, 0); }
        }
        if (ph == 2) {
          mfma_i(1, 1, 1);                      // (up, 1)
          if (more) {
            ld_a(b + 1, 1); dec_w(b + 1, 1); ld_ws(b + 1, 1);
            if (b == 0) ld_wr(1, 1);
          }
        }
        if (ph == 3 && more) {
          mfma_p(0);                            // gate's scale tiles of the next block
          mfma_i(0, 0, 0);                      // (gate, 0) of the next block
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i)
          res[x][ms][i] = __builtin_fmaf((float)I[slot][i], P[x][16 * ms + i], res[x][ms][i]);
        if ((b & 1) == 0) res[x][ms] = __builtin_amdgcn_mfma_f32_32x32x2f32(uop[ms], vop[x], res[x][ms], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    asm volatile("" : "+v"(res[0][0]), "+v"(res[0][1]), "+v"(res[1][0]), "+v"(res[1][1]));
    if (next) {
      store_scales(sr, st + 1, (st + 1) & 1);
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();
  }

  // ---- epilogue: lane = row n of the stream, accumulator i = slot 8 * (i / 4) + 4 * g + i % 4
  if constexpr (GU) {
    v16f hv[2];
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float gt = res[0][ms][i];
        hv[ms][i] = res[1][ms][i] * (gt / (1.0f + __expf(-gt)));
      }
    if constexpr (QUANT) {
      store_tile64_quant(lds, hv, H, N, m0, rows_valid, n0, S, hq, hsc, hbs);
      return;
    }
    if (store_tile64(lds, hv, H, N, 0, 0, m0, rows_valid, n0, N, nullptr, 0)) return;
    const int n = n0 + wave * 32 + l32;
    if (n < N) {
#pragma unroll
      for (int ms = 0; ms < 2; ++ms)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int r = ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          if (r >= rows_valid) continue;
          H[(size_t)(m0 + r) * N + n] = hv[ms][i];
        }
    }
  } else {
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int n = nx[x] + wave * 32 + l32;
      if (n >= N) continue;
#pragma unroll
      for (int ms = 0; ms < 2; ++ms)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int r = ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          if (r >= rows_valid) continue;
          float v = res[x][ms][i];
          float* cp = H + (size_t)(m0 + r) * ldc + c_off + n;
          if (accumulate == 1) {
            v += *cp;
          } else if (accumulate == 2) {
            const float gt = *cp;
            v *= gt / (1.0f + __expf(-gt));
          }
          *cp = v;
        }
    }
  }
}

// The gate / up tile on ready-made scale vectors in steps of 64 values (one 32-byte group of a row: two blocks), for
// three work-groups a compute unit: a stage is 17 KB where gemm4gu_body's is 34 (the quantizing epilogue's 36 KB set the array), and
// one scale tile and one pair of product tiles are live at a time -- the streams take turns inside a block -- so that the
// body stays within 168 registers.  The same products, scale tiles and min-term instructions in the same order per
// accumulator as gemm4gu_body (block 2s, the min term of blocks 2s and 2s + 1, block 2s + 1): the same bits.
// Stage: the 64 slots' int8 values [64][64] (16-byte piece c of row r at piece c ^ ((r / 4) % 4)), the two streams'
// packed rows [128][32] (piece c of row r at c ^ ((r / 8) % 2)), sa and sa * S [2][64], and per stream d * sc and
// -(dmin * mn) [2][128].  A wave brings per step: a quarter of the slots' rows, its 32 rows of both streams, one of
// the four token-side vectors (4-byte DMA, a lane a slot) and one of the four row-side vectors.
#define G5_STAGE 17408
#define G5_WQ0 4096
#define G5_WQ1 8192
#define G5_SA 12288
#define G5_U 12800
#define G5_WS0 13312
#define G5_V0 14336
#define G5_WS1 15360
#define G5_V1 16384
#define G5_LDS 36352  // (store_tile64_quant: 256 + 64 * 528 + 1024 + 1024)
__device__ __forceinline__ void gemm5gu_body(const uint8_t* __restrict__ rg, const uint8_t* __restrict__ ru,
                                             const signed char* __restrict__ aq, const float* __restrict__ asc,
                                             float* __restrict__ H, int M, int N, int K, size_t rows_total, size_t row_base,
                                             int m0, int rows_valid, int n0, const int* __restrict__ rowmap, int S,
                                             signed char* __restrict__ hq, float* __restrict__ hsc, short* __restrict__ hbs,
                                             const float* __restrict__ au, const float* __restrict__ wsg,
                                             const float* __restrict__ wsu, float* __restrict__ hu) {
  static_assert(2 * G5_STAGE <= G5_LDS, "two stages fit the epilogue's array");
  __shared__ alignas(16) uint8_t lds[G5_LDS];
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  const PlanesQ4K pl = planes_q4k(rows_total, nsb);
  auto token_row = [&](int r) { return rowmap[m0 + (r < rows_valid ? r : 0)]; };  // slots past the tile read its first

  // ---- what this lane fetches each step
  const int Ra = 16 * wave + (lane >> 2), Rw = 32 * wave + (lane >> 1);
  uint32_t aoff = (uint32_t)token_row(Ra) * (uint32_t)K + 16u * ((lane & 3) ^ ((Ra >> 2) & 3));
  uint32_t woff = (uint32_t)min(n0 + Rw, N - 1) * (uint32_t)nsb * 128u + 16u * ((lane & 1) ^ ((Rw >> 3) & 1));
  const uint8_t* wg0 = rg + pl.qs + row_base * nsb * 128;
  const uint8_t* wu0 = ru + pl.qs + row_base * nsb * 128;
  // token side: waves 0, 1 sa of blocks 0, 1; waves 2, 3 sa * S of blocks 0, 1.  Row side: wave w vector w of
  // (gate d * sc, gate -(dmin * mn), up d * sc, up -(dmin * mn)): lane l the rows 4 (l % 32) .. + 3 of block l / 32
  uint32_t toff = (uint32_t)token_row(lane) * 4u;
  const uint8_t* tbase = (const uint8_t*)(wave < 2 ? asc : au) + (size_t)(wave & 1) * M * 4;
  const uint8_t* rbase = (const uint8_t*)((wave >> 1) ? wsu : wsg) + ((wave & 1) ? (size_t)(K >> 5) * rows_total * 4 : (size_t)0);
  uint32_t roff = ((uint32_t)(lane >> 5) * (uint32_t)rows_total + (uint32_t)row_base + (uint32_t)n0 + 4u * (lane & 31)) * 4u;

  auto dma_step = [&](int st, int stage) {
    uint8_t* base = lds + stage * G5_STAGE;
    asm volatile("" : "+v"(aoff), "+v"(woff), "+v"(toff), "+v"(roff));  // (addresses formed here, not kept over the loop)
    g3_dma16(aq + (size_t)st * 64 + aoff, base + wave * 1024);
    g3_dma16(wg0 + (size_t)st * 32 + woff, base + G5_WQ0 + wave * 1024);
    g3_dma16(wu0 + (size_t)st * 32 + woff, base + G5_WQ1 + wave * 1024);
    g3_dma4(tbase + (size_t)st * 2 * M * 4 + toff, base + G5_SA + wave * 256);
    g3_dma16(rbase + (size_t)st * 2 * rows_total * 4 + roff, base + G5_WS0 + wave * 1024);
  };

  // ---- operand addresses of this lane (bytes from a stage's start)
  int oa[2];
#pragma unroll
  for (int b = 0; b < 2; ++b) oa[b] = l32 * 64 + (((2 * b + g) ^ ((l32 >> 2) & 3)) * 16);
  const int ow = (wave * 32 + l32) * 32 + ((g ^ ((l32 >> 3) & 1)) * 16);

  v16f res[2][2];  // [gate / up][slot tile]
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int i = 0; i < 16; ++i) res[x][ms][i] = 0.0f;

  const int steps = 4 * nsb;
  dma_step(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the stage has landed
  __syncthreads();

  // TWO = false: a tile of at most 32 slots; its second slot tile, all padding, is left out (half the products and
  // their sums).  Two loops, chosen once per tile: with the choice as a branch inside one loop the compiler kept both
  // forms' values live and spilled 20 registers.
  auto loop = [&](auto two_c) {
    constexpr bool TWO = decltype(two_c)::value;
#pragma unroll 1
    for (int st = 0; st < steps; ++st) {
      const uint8_t* Sb = lds + (st & 1) * G5_STAGE;
      if (st + 1 < steps) dma_step(st + 1, (st + 1) & 1);
      // (every operand of the step is read here, in one go: the reads' latency is paid once a step, not once a block
      //  and stream)
      v4i wr[2];
      wr[0] = *(const v4i*)(Sb + G5_WQ0 + ow);
      wr[1] = *(const v4i*)(Sb + G5_WQ1 + ow);
      v4i a16s[2][2];
      float saops[2], wsops[2][2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        a16s[b][0] = *(const v4i*)(Sb + oa[b]);
        if constexpr (TWO) a16s[b][1] = *(const v4i*)(Sb + oa[b] + 32 * 64);
        saops[b] = ((const float*)(Sb + G5_SA))[b * 64 + lane];
#pragma unroll
        for (int x = 0; x < 2; ++x) wsops[b][x] = ((const float*)(Sb + (x ? G5_WS1 : G5_WS0)))[b * 128 + wave * 32 + l32];
      }
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const v4i* a16 = a16s[b];
        const float saop = saops[b];
#pragma unroll
        for (int x = 0; x < 2; ++x) {
          const float wsop = wsops[b][x];
          v4i w16;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t v = (uint32_t)wr[x][i];
            w16[i] = (int)(b ? (v >> 4) & 0x0F0F0F0Fu : v & 0x0F0F0F0Fu);
          }
          v32f zf;
#pragma unroll
          for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
          v16i z;
#pragma unroll
          for (int i = 0; i < 16; ++i) z[i] = 0;
          const v32f P = __builtin_amdgcn_mfma_f32_32x32x1f32(saop, wsop, zf, 0, 0, 0);
          const v16i I0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[0], w16, z, 0, 0, 0);
          v16i I1;
          if constexpr (TWO) I1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[1], w16, z, 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = 0; i < 16; ++i) res[x][0][i] = __builtin_fmaf((float)I0[i], P[i], res[x][0][i]);
          if constexpr (TWO) {
#pragma unroll
            for (int i = 0; i < 16; ++i) res[x][1][i] = __builtin_fmaf((float)I1[i], P[16 + i], res[x][1][i]);
          }
          if (b == 0) {  // min term of the step's two blocks: lane half g supplies block g
            const float vop = ((const float*)(Sb + (x ? G5_V1 : G5_V0)))[g * 128 + wave * 32 + l32];
#pragma unroll
            for (int ms = 0; ms < (TWO ? 2 : 1); ++ms) {
              const float uop = ((const float*)(Sb + G5_U))[g * 64 + ms * 32 + l32];
              res[x][ms] = __builtin_amdgcn_mfma_f32_32x32x2f32(uop, vop, res[x][ms], 0, 0, 0);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      asm volatile("" : "+v"(res[0][0]), "+v"(res[0][1]), "+v"(res[1][0]), "+v"(res[1][1]));
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
    }
  };
  if (rows_valid > 32) loop(std::true_type{});
  else loop(std::false_type{});

  // ---- epilogue: lane = row n of the stream, accumulator i = slot 8 * (i / 4) + 4 * g + i % 4
  v16f hv[2];
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float gt = res[0][ms][i];
      hv[ms][i] = res[1][ms][i] * (gt / (1.0f + __expf(-gt)));
    }
  store_tile64_quant(lds, hv, H, N, m0, rows_valid, n0, S, hq, hsc, hbs, hu);
}

// -DQUANT=1 -DPRE=2: the -DQUANT=1 kernel's arguments and, behind them, au [K/32][M] = sa * S of the chunk's tokens, the
// two tensors' ws | v from q4k_wscales (made when the layer is uploaded), and hu
// [F/32][S] (may be null): the expert inputs' sa * S, written by the quantizing epilogue for the down kernel's -DPRE=1 form
extern "C" __global__ __launch_bounds__(256, 3) void moe_gateup_q__QT12_QUANT1_PRE2(
    const uint8_t* rg, const uint8_t* ru, int F, int K, const uint32_t* tabs, const signed char* aq, const float* asc,
    int M, const int* tiles, const int* stok, float* h, const short* absum, int S, signed char* hq, float* hsc,
    short* hbs, const float* au, const float* wsg, const float* wsu, float* hu, int NE) {
  int ti, chunk;
  if (!moe_tile_of(tiles[0], gridDim.x, ti, chunk)) return;
  const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];
  gemm5gu_body(rg, ru, aq, asc, h, M, F, K, (size_t)NE * F, (size_t)e * F, r0, min(nr, G6_BM), chunk * BN, stok, S, hq, hsc,
               hbs, au, wsg, wsu, hu);
}

// moe_gateup_q: arguments as the reference's (zero/kernels/decode_moe.cl:92-94) -- the two raw expert tensors
// [NE][F][K], the tile list (tiles of at most 64 slots), stok = the token row of every slot, h [slots][F] -- and, as its
// extra arguments, the activations' sums per 16 values.  grid (ceil(F / 128) * 256, tile work-groups: the most tiles
// there can be, rounded up to a multiple of 8): one tile and row chunk a work-group, dealt by moe_tile_of.
extern "C" __global__ __launch_bounds__(256, 2) void moe_gateup_q__QT12(
    const uint8_t* rg, const uint8_t* ru, int F, int K, const uint32_t* tabs, const signed char* aq, const float* asc,
    int M, const int* tiles, const int* stok, float* h, const short* absum, int NE) {
  int ti, chunk;
  if (!moe_tile_of(tiles[0], gridDim.x, ti, chunk)) return;
  const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];
  gemm4gu_body<true>(rg, ru, aq, asc, absum, h, M, F, K, (size_t)NE * F, (size_t)e * F, r0, min(nr, G6_BM), chunk * BN, stok,
                     0, 0, 0);
}
// -DQUANT=1: with the expert inputs' quantization done on the way out (store_tile64_quant): h as before and
// hq [S][F], hsc [F/32][S], hbs [F/16][S], what moe_quant_sums would make of h, bit for bit.  F a multiple of 128.
extern "C" __global__ __launch_bounds__(256, 2) void moe_gateup_q__QT12_QUANT1(
    const uint8_t* rg, const uint8_t* ru, int F, int K, const uint32_t* tabs, const signed char* aq, const float* asc,
    int M, const int* tiles, const int* stok, float* h, const short* absum, int S, signed char* hq, float* hsc,
    short* hbs, int NE) {
  int ti, chunk;
  if (!moe_tile_of(tiles[0], gridDim.x, ti, chunk)) return;
  const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];
  gemm4gu_body<true, true>(rg, ru, aq, asc, absum, h, M, F, K, (size_t)NE * F, (size_t)e * F, r0, min(nr, G6_BM), chunk * BN,
                           stok, 0, 0, 0, S, hq, hsc, hbs);
}

// ---------------------------------------------------------------------------------------------------------------
// Q8_0, dense, 64-token tiles: the shape of the Q6_K kernel for matrices with few 128 x 128 tiles (4096 x 4096 at 512
// tokens is 128 of them on 256 compute units; in 64-token tiles it is 256).  The int8 rows go straight into LDS and
// into the products unchanged; res += (sa[m][b] * d[n][b]) * (float)I.
#define G8_STAGE 27648
#define G8_W 8192
#define G8_SA 24576
#define G8_WS 25600

__device__ __forceinline__ void gemm8_body(const uint8_t* __restrict__ raw, const signed char* __restrict__ aq,
                                  const float* __restrict__ asc, float* __restrict__ C, int M, int N, int K, int ldc,
                                  int c_off, int accumulate, int s_begin, int s_end, int m0, int rows_valid, int n0) {
  __shared__ alignas(16) uint8_t lds[2 * G8_STAGE];
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  const PlanesQ80 pl = planes_q80((size_t)N, nsb);
  auto token_row = [&](int r) { return m0 + (r < rows_valid ? r : 0); };  // rows past the tile read its first row

  // activations: 2 instructions a wave, 8 rows each; weights: 4 instructions a wave, 8 rows of 128 bytes each
  uint32_t aoff[2], woff[4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
    aoff[i] = (uint32_t)token_row((wave * 2 + i) * 8 + (lane >> 3)) * (uint32_t)K + 16u * ((lane & 7) ^ (lane >> 3));
#pragma unroll
  for (int i = 0; i < 4; ++i)
    woff[i] = (uint32_t)min(n0 + (wave * 4 + i) * 8 + (lane >> 3), N - 1) * (uint32_t)nsb * 256u + 16u * ((lane & 7) ^ (lane >> 3));
  const signed char* abase = aq + (size_t)s_begin * 256;
  const uint8_t* wbase = raw + pl.qs + (size_t)s_begin * 256;
  // scales: thread t prepares token t % 64, block t / 64 of the step, and weight row t / 2, blocks 2 (t % 2) + {0, 1}
  const int r_s = t & 63, b_s = wave;
  const bool tok_valid = r_s < rows_valid;
  const uint32_t m_s = (uint32_t)token_row(r_s);
  const int n_s = min(n0 + (t >> 1), N - 1), p_s = t & 1;

  auto dma_step = [&](int st, int stage) {
    uint8_t* base = lds + stage * G8_STAGE;
    const signed char* ab = abase + (size_t)st * 128;
    const uint8_t* wb = wbase + (size_t)st * 128;
#pragma unroll
    for (int i = 0; i < 2; ++i) asm volatile("" : "+v"(aoff[i]));
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(woff[i]));
#pragma unroll
    for (int i = 0; i < 2; ++i) g3_dma16(ab + aoff[i], base + (wave * 2 + i) * 1024);
#pragma unroll
    for (int i = 0; i < 4; ++i) g3_dma16(wb + woff[i], base + G8_W + (wave * 4 + i) * 1024);
  };
  float sa_r;
  uint32_t d_r;
  auto load_scales = [&](int st) {
    sa_r = (asc + (size_t)(s_begin * 8 + st * 4 + b_s) * M)[m_s];
    d_r = *(const uint32_t*)(raw + pl.d + (((size_t)n_s * nsb + s_begin) * 8 + st * 4 + 2 * p_s) * 2);
  };
  auto store_scales = [&](int stage) {
    uint8_t* base = lds + stage * G8_STAGE;
    ((float*)(base + G8_SA))[b_s * 64 + r_s] = tok_valid ? sa_r : 0.0f;
    ((float*)(base + G8_WS))[(2 * p_s) * 128 + (t >> 1)] = f16_bits_to_f32(d_r);
    ((float*)(base + G8_WS))[(2 * p_s + 1) * 128 + (t >> 1)] = f16_bits_to_f32(d_r >> 16);
  };

  int oa[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) oa[b] = l32 * 128 + (((2 * b + g) ^ (l32 & 7)) * 16);
  const int wrow = G8_W + wave * 32 * 128;

  v16f res[2];
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int i = 0; i < 16; ++i) res[ms][i] = 0.0f;

  const int steps = 2 * (s_end - s_begin);
  if (steps > 0) {
    dma_step(0, 0);
    load_scales(0);
    store_scales(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the stage has landed
  }
  __syncthreads();

#pragma unroll 1
  for (int st = 0; st < steps; ++st) {
    const uint8_t* Sb = lds + (st & 1) * G8_STAGE;
    const bool next = st + 1 < steps;
    if (next) {
      dma_step(st + 1, (st + 1) & 1);
      load_scales(st + 1);
    }
    v4i a16[2][2], w16[2];  // [buffer][ms]; [buffer]
    float saop[2], wsop[2];
    v32f P[2];
    v16i I[2];
    auto ld_ops = [&](int b, int buf) {
      a16[buf][0] = *(const v4i*)(Sb + oa[b]);
      a16[buf][1] = *(const v4i*)(Sb + oa[b] + 32 * 128);
      w16[buf] = *(const v4i*)(Sb + wrow + oa[b]);
      saop[buf] = ((const float*)(Sb + G8_SA))[b * 64 + lane];
      wsop[buf] = ((const float*)(Sb + G8_WS))[b * 128 + wave * 32 + l32];
    };
    auto mfma_p = [&](int buf) {
      v32f zf;
#pragma unroll
      for (int i = 0; i < 32; ++i) zf[i] = 0.0f;
      P[buf] = __builtin_amdgcn_mfma_f32_32x32x1f32(saop[buf], wsop[buf], zf, 0, 0, 0);
    };
    auto mfma_i = [&](int buf, int ms, int slot) {
      v16i z;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] = 0;
      I[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a16[buf][ms], w16[buf], z, 0, 0, 0);
    };
    ld_ops(0, 0);
    mfma_p(0);
    mfma_i(0, 0, 0);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int buf = b & 1;
      const bool more = b + 1 < 4;
#pragma unroll
      for (int ms = 0; ms < 2; ++ms) {
        if (ms == 0) {
          mfma_i(buf, 1, 1);
          if (more) ld_ops(b + 1, buf ^ 1);
        } else if (more) {
          mfma_p(buf ^ 1);
          mfma_i(buf ^ 1, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i) res[ms][i] = __builtin_fmaf((float)I[ms][i], P[buf][16 * ms + i], res[ms][i]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    asm volatile("" : "+v"(res[0]), "+v"(res[1]));  // (the sums are complete before the branches below)
    if (next) {
      store_scales((st + 1) & 1);
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();
  }

  const int n = n0 + wave * 32 + l32;
  if (n < N) {
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = ms * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
        if (r >= rows_valid) continue;
        float v = res[ms][i];
        float* cp = C + (size_t)(m0 + r) * ldc + c_off + n;
        if (accumulate == 1) {
          v += *cp;
        } else if (accumulate == 2) {
          const float gt = *cp;
          v *= gt / (1.0f + __expf(-gt));
        }
        *cp = v;
      }
  }
}

// Tile of work-group `id` out of mt x nt tiles.  XCDs take work-groups in turn (id % 8), each running 64 at a time:
// those 64 are made an 8 x 8 block of tiles when both tile counts are multiples of 8 and the blocks share out evenly
// over the 8 XCDs.  Any other shape: the tiles are put in the order "panels of 8 token tiles; within a panel row tile
// by row tile" and that list is cut into 8 runs, one per XCD (XCD x's j-th work-group takes the j-th tile of run x), so
// that the 64 tiles an XCD works on are 8 token tiles x 8 row tiles whose successors keep the same token tiles: the
// panel's activations stay in the XCD's L2 while the weight rows stream through it once per panel.  (Token tiles
// fastest over the whole grid, as it was, gave every XCD 4 token tiles x 16 row tiles and every row tile to all 8 XCDs:
// the 151936 x 5120 Q6_K head at 2048 tokens read 6.9 GB from memory for 0.65 GB of input.)
__device__ inline void tile_of(int id, int mt, int nt, int& tm, int& tn) {
  if ((mt & 7) == 0 && (nt & 7) == 0 && (((mt >> 3) * (nt >> 3)) & 7) == 0) {  // (whole 8 x 8 blocks, 8 XCDs' worth)
    const int x = id & 7, q = id >> 3;
    const int st = (q >> 6) * 8 + x, within = q & 63;
    const int smt = mt >> 3;
    tm = (st % smt) * 8 + (within & 7);
    tn = (st / smt) * 8 + (within >> 3);
  } else {
    const int total = mt * nt, x = id & 7, j = id >> 3;
    const int L = x * (total >> 3) + min(x, total & 7) + j;  // (XCD y has total / 8 tiles, one more if y < total % 8)
    const int panel = L / (8 * nt), rem = L - panel * 8 * nt, pw = min(8, mt - panel * 8);
    tn = rem / pw;
    tm = panel * 8 + rem - tn * pw;
  }
}

// gemm, dense.  Arguments as the reference's (zero/kernels/gemm.cl:163-166); with the weights decoded in the kernel
// its (wq, wh) pair is (raw planes, unused), absum is unused (the block sums are taken from the int8 values), and
// rgroup (its cache-blocking knob) is accepted and ignored.  grid: ceil(N / 128) * ceil(M / 128) work-groups of 256.
#define GEMM2_INST(QT)                                                                                               \
  extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE##QT##_ACT321(                                      \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {        \
    const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;                                                         \
    int tm, tn;                                                                                                       \
    tile_of(blockIdx.x, mt, nt, tm, tn);                                                                              \
    const int m0 = tm * BM, n0 = tn * BN;                                                                             \
    gemm2_body<QT, false>(raw, aq, asc, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,         \
                          min(BM, M - m0), n0, nullptr, 0, nullptr, 0);                                               \
  }

// gemm over expert tiles (reference zero/kernels/gemm.cl:146-161, -DMOE_TILES): W holds all experts' rows (N each);
// tile t of the list = (expert, first slot, rows <= 128) from moe_scan; slot r reads token row rowmap[r] (use_map) or
// r, writes C row r, times rowscale[r] (use_scale).  Experts [e0, e1).  grid (ceil(N / 128), tile work-groups >= the
// tiles of those experts): one tile and row chunk a work-group, dealt by moe_tile_of.
#define GEMM2_TILES_INST(QT)                                                                                         \
  extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE##QT##_ACT321_MOE_TILES1(                           \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int accumulate, const int* tiles, const int* tstart, int e0, int e1,    \
      const int* rowmap, int use_map, const float* rowscale, int use_scale, int NE) {                                 \
    /* one tile a work-group (grid.y covers the most tiles there can be, as the reference launches it,              \
       zero/engine_moe.h:153): as a loop over tiles the body spilled 15-45 registers */                              \
    int ti, chunk;                                                                                                    \
    if (!moe_tile_of(tstart[e1] - tstart[e0], gridDim.x, ti, chunk)) return;                                          \
    ti += tstart[e0];                                                                                                 \
    const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];                                  \
    gemm2_body<QT, true>(raw, aq, asc, C, M, N, K, ldc, 0, accumulate, 0, K >> 8, (size_t)NE * N, (size_t)e * N, r0,  \
                         min(nr, BM), chunk * BN, rowmap, use_map, rowscale, use_scale);                              \
  }

GEMM2_INST(8)
GEMM2_TILES_INST(8)
// Q5_K: the DMA-staged bodies below (the Q4_K arithmetic on values 0..31)
// IQ4_XS: the register-staged body too (codes to values through the table as they are stored to LDS)
GEMM2_INST(23)
GEMM2_TILES_INST(23)
// Q4_0: the same body (nibbles to values as they are stored to LDS, a block's f16 scale as Q8_0's)
GEMM2_INST(2)
GEMM2_TILES_INST(2)
// IQ4_NL, MXFP4: Q4_0's path with the nibbles through the types' tables (MXFP4: a block's scale from its E8M0 byte)
GEMM2_INST(20)
GEMM2_TILES_INST(20)
GEMM2_INST(39)
GEMM2_TILES_INST(39)
// Q4_K -DBM=64: 64 tokens x 256 rows per work-group (grid ceil(N / 256) * ceil(M / 64) work-groups), K from 0
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_BM64(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + 255) / 256;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * 256;
  gemm4gu_body<false>(raw, raw, aq, asc, absum, C, M, N, K, (size_t)N, 0, m0, min(G6_BM, M - m0), n0, nullptr, ldc, c_off,
                      accumulate);
}
// Q4_K -DBM=64 -DBN=128: 64 tokens x 128 rows per work-group (grid ceil(N / 128) * ceil(M / 64)): the expert-tile body on
// the dense matrix, for chunks so short that the larger tiles leave most compute units without a work-group
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_BM64_BN128(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  gemm4_body(raw, aq, asc, absum, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0, min(G6_BM, M - m0),
             n0, nullptr, 0, nullptr, 0);
}
// -DPRE64=1: the same tiles on ready-made scale vectors (gemm4_body's PRE; the arguments of the -DAU=2 kernel: au in the
// place of the unused plane pointer, wsv = ws | v in the place of the block sums), three work-groups a compute unit
extern "C" __global__ __launch_bounds__(256, 3) void gemm__QTYPE12_ACT321_BM64_BN128_PRE641(
    const uint8_t* raw, const float* au, const signed char* aq, const float* asc, const float* wsv, float* C, int M, int N,
    int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  gemm4_body<true, QT_Q4_K, true>(raw, aq, asc, nullptr, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                                  min(G6_BM, M - m0), n0, nullptr, 0, nullptr, 0, au, wsv);
}
// The same with K shared out over gridDim.y work-groups per tile (-DSPLITK): work-group (x, y) takes the y-th of
// gridDim.y even pieces of superblocks [s_begin, s_end) and stores its partial tile in slice y of C, here a workspace
// [gridDim.y][M][ldc] (c_off and accumulate apply in splitk_reduce, which adds the slices in order).  A chunk of 64
// tokens gives 136 tiles for 256 compute units, and a tile's work-group needs 75 us to walk through K = 5120 alone.
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_BM64_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm4_body<true>(raw, aq, asc, absum, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,
                   s_begin + ns * (y + 1) / ny, (size_t)N, 0, m0, min(G6_BM, M - m0), n0, nullptr, 0, nullptr, 0);
}
// (-DBM=32: chunks of at most 32 rows, M <= 32: one slot tile.  A kernel of its own: the body's LDS is a static array
//  per instantiation, and two in one kernel would halve the work-groups a compute unit holds)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_BM32_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int n0 = blockIdx.x * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm4_body<false>(raw, aq, asc, absum, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,
                    s_begin + ns * (y + 1) / ny, (size_t)N, 0, 0, min(32, M), n0, nullptr, 0, nullptr, 0);
}
// (the same two for Q5_K)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE13_ACT321_BM64_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm4_body<true, QT_Q5_K>(raw, aq, asc, absum, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,
                            s_begin + ns * (y + 1) / ny, (size_t)N, 0, m0, min(G6_BM, M - m0), n0, nullptr, 0, nullptr, 0);
}
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE13_ACT321_BM32_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int n0 = blockIdx.x * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm4_body<false, QT_Q5_K>(raw, aq, asc, absum, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,
                             s_begin + ns * (y + 1) / ny, (size_t)N, 0, 0, min(32, M), n0, nullptr, 0, nullptr, 0);
}
// (-DBM=128 -DBN=128 -DSPLITK: the same over the 128 x 128 tiles of the dense kernel, for 65-128 tokens)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_BM128_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm3_body<false>(raw, aq, asc, absum, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,
                    s_begin + ns * (y + 1) / ny, (size_t)N, 0, m0, min(BM, M - m0), n0, nullptr, 0, nullptr, 0);
}
// (Q8_0 -DBM=64 -DBN=128 -DSPLITK: the 64-token form's tiles)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE8_ACT321_BM64_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm8_body(raw, aq, asc, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny, s_begin + ns * (y + 1) / ny,
             m0, min(G6_BM, M - m0), n0);
}
// (Q6_K -DBM=64 -DBN=128 -DSPLITK: its dense kernel's tiles)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE14_ACT321_BM64_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm6_body<false>(raw, aq, asc, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny, s_begin + ns * (y + 1) / ny,
             m0, min(G6_BM, M - m0), n0);
}
// (... -DHDS=1 / 2: planes written out from IQ3_XXS / IQ3_S, gemm6_body<..., HD>)
#define GEMM6_HDS_INST(HDV)                                                                                          \
  extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE14_ACT321_BM64_BN128_SPLITK1_HDS##HDV(               \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {        \
    const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;                                                   \
    int tm, tn;                                                                                                       \
    tile_of(blockIdx.x, mt, nt, tm, tn);                                                                              \
    const int m0 = tm * G6_BM, n0 = tn * BN;                                                                          \
    const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;                                                   \
    gemm6_body<false, HDV>(raw, aq, asc, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,           \
                           s_begin + ns * (y + 1) / ny, m0, min(G6_BM, M - m0), n0);                                   \
  }
GEMM6_HDS_INST(1)
GEMM6_HDS_INST(2)
// (Q5_K, IQ4_XS -DBM=128 -DBN=128 -DSPLITK: the register-staged body's tiles)
#define GEMM2_SPLITK_INST(QT)                                                                                        \
  extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE##QT##_ACT321_BM128_BN128_SPLITK1(                  \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {        \
    const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;                                                         \
    int tm, tn;                                                                                                       \
    tile_of(blockIdx.x, mt, nt, tm, tn);                                                                              \
    const int m0 = tm * BM, n0 = tn * BN;                                                                             \
    const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;                                                   \
    gemm2_body<QT, false>(raw, aq, asc, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,           \
                          s_begin + ns * (y + 1) / ny, (size_t)N, 0, m0, min(BM, M - m0), n0, nullptr, 0, nullptr, 0); \
  }
GEMM2_SPLITK_INST(23)
GEMM2_SPLITK_INST(2)
GEMM2_SPLITK_INST(20)
GEMM2_SPLITK_INST(39)
// (Q5_K: the DMA-staged body, as Q4_K)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE13_ACT321_BM128_BN128_SPLITK1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int ns = s_end - s_begin, y = blockIdx.y, ny = gridDim.y;
  gemm3_body<false, QT_Q5_K>(raw, aq, asc, absum, C + (size_t)y * M * ldc, M, N, K, ldc, 0, 0, s_begin + ns * y / ny,
                             s_begin + ns * (y + 1) / ny, (size_t)N, 0, m0, min(BM, M - m0), n0, nullptr, 0, nullptr, 0);
}
// splitk_reduce: C[m][c_off + n] (=, +=, silu(C) *) sum over the ny slices of ws [ny][M][N], slice 0 first.
// grid: ceil(M * N / 256) work-groups of 256.
extern "C" __global__ __launch_bounds__(256) void splitk_reduce(const float* __restrict__ ws, int ny, float* C, int M, int N,
                                                                int ldc, int c_off, int accumulate) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, total = (size_t)M * N;
  if (i >= total) return;
  float v = ws[i];
  for (int y = 1; y < ny; ++y) v += ws[(size_t)y * total + i];
  const size_t m = i / (size_t)N, n = i - m * (size_t)N;
  float* cp = C + m * ldc + c_off + n;
  if (accumulate == 1) {
    v += *cp;
  } else if (accumulate == 2) {
    const float gt = *cp;
    v *= gt / (1.0f + __expf(-gt));
  }
  *cp = v;
}
// -DBM=64: the 64-token form (grid ceil(N / 128) * ceil(M / 64) work-groups)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE8_ACT321_BM64(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  gemm8_body(raw, aq, asc, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, m0, min(G6_BM, M - m0), n0);
}

extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  gemm3_body<false>(raw, aq, asc, absum, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                    min(BM, M - m0), n0, nullptr, 0, nullptr, 0);
}
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE13_ACT321(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  gemm3_body<false, QT_Q5_K>(raw, aq, asc, absum, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                             min(BM, M - m0), n0, nullptr, 0, nullptr, 0);
}
// -DAU: the same two kernels with the token side's scale vectors ready-made (gemm3_body<..., AU>): the second argument,
// unused otherwise, is au[K / 32][M] = sa * S; M a multiple of 4.  No counterpart in the reference.
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_AU1(
    const uint8_t* raw, const uint8_t* au, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  gemm3_body<false, QT_Q4_K, 1>(raw, aq, asc, absum, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                                min(BM, M - m0), n0, nullptr, 0, nullptr, 0, (const float*)au);
}
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE13_ACT321_AU1(
    const uint8_t* raw, const uint8_t* au, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  gemm3_body<false, QT_Q5_K, 1>(raw, aq, asc, absum, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                                min(BM, M - m0), n0, nullptr, 0, nullptr, 0, (const float*)au);
}
// -DAU=2: the row side's scale vectors ready-made as well: wsv (q4k_wscales) stands in absum's place, which the kernel
// no longer reads.  N a multiple of 4.
#define GEMM3_AU2_INST(QT)                                                                                           \
  extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE##QT##_ACT321_AU2(                                  \
      const uint8_t* raw, const uint8_t* au, const signed char* aq, const float* asc, const short* wsv, float* C,     \
      int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {                  \
    const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;                                                         \
    int tm, tn;                                                                                                       \
    tile_of(blockIdx.x, mt, nt, tm, tn);                                                                              \
    const int m0 = tm * BM, n0 = tn * BN;                                                                             \
    gemm3_body<false, QT, 2>(raw, aq, asc, nullptr, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, \
                             m0, min(BM, M - m0), n0, nullptr, 0, nullptr, 0, (const float*)au, (const float*)wsv);   \
  }
GEMM3_AU2_INST(12)
GEMM3_AU2_INST(13)
// -DAU=3: Q4_K with the min term on the bf16 matrix instruction: au and wsv hold the operands' pieces (act_usum_bf16,
// q4k_wscales_bf16).  M even, N a multiple of 4.
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_AU3(
    const uint8_t* raw, const uint8_t* au, const signed char* aq, const float* asc, const short* wsv, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  gemm3_body<false, QT_Q4_K, 3>(raw, aq, asc, nullptr, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                                min(BM, M - m0), n0, nullptr, 0, nullptr, 0, (const float*)au, (const float*)wsv);
}
// -DAU=3 -DWM=4: the same in tiles of 256 tokens x 128 rows, work-groups of 512 threads (gemm3_body's WM).
extern "C" __global__ __launch_bounds__(512, 2) void gemm__QTYPE12_ACT321_AU3_WM4(
    const uint8_t* raw, const uint8_t* au, const signed char* aq, const float* asc, const short* wsv, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + 255) / 256, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * 256, n0 = tn * BN;
  gemm3_body<false, QT_Q4_K, 3, 4>(raw, aq, asc, nullptr, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                                   min(256, M - m0), n0, nullptr, 0, nullptr, 0, (const float*)au, (const float*)wsv);
}
// -DAU=4: the -DAU=3 form for chunks whose activation scales are per 256 values (asc holds each eight times): wsv holds
// the integer sub-block scales as int32 [K / 32][N], the min term's pieces as before, then d as f32 [K / 256][N]
// (q4k_wscales_int).
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_AU4(
    const uint8_t* raw, const uint8_t* au, const signed char* aq, const float* asc, const short* wsv, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  gemm3_body<false, QT_Q4_K, 4>(raw, aq, asc, nullptr, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, (size_t)N, 0, m0,
                                min(BM, M - m0), n0, nullptr, 0, nullptr, 0, (const float*)au, (const float*)wsv);
}
// (tiles of at most 64 slots: the engine builds the tile list for that size)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE12_ACT321_MOE_TILES1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int accumulate, const int* tiles, const int* tstart, int e0, int e1, const int* rowmap,
    int use_map, const float* rowscale, int use_scale, int NE) {
  int ti, chunk;  // one tile and row chunk a work-group (as a loop over tiles the body spilled registers)
  if (!moe_tile_of(tstart[e1] - tstart[e0], gridDim.x, ti, chunk)) return;
  ti += tstart[e0];
  const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];
  gemm4_body<true>(raw, aq, asc, absum, C, M, N, K, ldc, 0, accumulate, 0, K >> 8, (size_t)NE * N, (size_t)e * N, r0,
                   min(nr, G6_BM), chunk * BN, rowmap, use_map, rowscale, use_scale);
}

// -DPRE=1: the scale vectors ready-made (gemm4_body's PRE): au [K/32][M] from act_usum over the slots' scales and sums,
// wsv the tensor's ws | v from q4k_wscales (made when the layer is uploaded).  Without the scale registers the body fits
// 168 registers, three work-groups a compute unit (one register spilled outside the loop): the down projection of 32768
// slots x 768 -> 2048 in 0.220 ms against 0.247 with two (the plain form spills six at that size and gains nothing).
extern "C" __global__ __launch_bounds__(256, 3) void gemm__QTYPE12_ACT321_MOE_TILES1_PRE1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int accumulate, const int* tiles, const int* tstart, int e0, int e1, const int* rowmap,
    int use_map, const float* rowscale, int use_scale, const float* au, const float* wsv, int NE) {
  int ti, chunk;
  if (!moe_tile_of(tstart[e1] - tstart[e0], gridDim.x, ti, chunk)) return;
  ti += tstart[e0];
  const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];
  gemm4_body<true, QT_Q4_K, true>(raw, aq, asc, absum, C, M, N, K, ldc, 0, accumulate, 0, K >> 8, (size_t)NE * N,
                                  (size_t)e * N, r0, min(nr, G6_BM), chunk * BN, rowmap, use_map, rowscale, use_scale, au,
                                  wsv);
}

// (Q5_K experts: the same body, one tile of at most 64 slots per work-group)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE13_ACT321_MOE_TILES1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int accumulate, const int* tiles, const int* tstart, int e0, int e1, const int* rowmap,
    int use_map, const float* rowscale, int use_scale, int NE) {
  int ti, chunk;
  if (!moe_tile_of(tstart[e1] - tstart[e0], gridDim.x, ti, chunk)) return;
  ti += tstart[e0];
  const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];
  gemm4_body<true, QT_Q5_K>(raw, aq, asc, absum, C, M, N, K, ldc, 0, accumulate, 0, K >> 8, (size_t)NE * N, (size_t)e * N,
                            r0, min(nr, G6_BM), chunk * BN, rowmap, use_map, rowscale, use_scale);
}

// Q6_K: the dense form has its own body (64-token tiles: grid ceil(N / 128) * ceil(M / 64) work-groups); the form over
// expert tiles runs the plain kernel.
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE14_ACT321(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {
  const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, mt, nt, tm, tn);
  const int m0 = tm * G6_BM, n0 = tn * BN;
  gemm6_body<false>(raw, aq, asc, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, m0, min(G6_BM, M - m0), n0);
}
// (-DHD=1 / 2, -DHDT=1 / 2: planes written out from IQ3_XXS / IQ3_S, gemm6_body<..., HD>)
#define GEMM6_HD_INST(HDV)                                                                                           \
  extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE14_ACT321_HD##HDV(                                   \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int c_off, int accumulate, int rgroup, int s_begin, int s_end) {        \
    const int mt = (M + G6_BM - 1) / G6_BM, nt = (N + BN - 1) / BN;                                                   \
    int tm, tn;                                                                                                       \
    tile_of(blockIdx.x, mt, nt, tm, tn);                                                                              \
    const int m0 = tm * G6_BM, n0 = tn * BN;                                                                          \
    gemm6_body<false, HDV>(raw, aq, asc, C, M, N, K, ldc, c_off, accumulate, s_begin, s_end, m0, min(G6_BM, M - m0),   \
                           n0);                                                                                       \
  }                                                                                                                   \
  extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE14_ACT321_MOE_TILES1_HDT##HDV(                       \
      const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum,      \
      float* C, int M, int N, int K, int ldc, int accumulate, const int* tiles, const int* tstart, int e0, int e1,    \
      const int* rowmap, int use_map, const float* rowscale, int use_scale, int NE) {                                 \
    int ti, chunk;                                                                                                    \
    if (!moe_tile_of(tstart[e1] - tstart[e0], gridDim.x, ti, chunk)) return;                                          \
    ti += tstart[e0];                                                                                                 \
    const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];                                  \
    gemm6_body<true, HDV>(raw, aq, asc, C, M, N, K, ldc, 0, accumulate, 0, K >> 8, r0, min(nr, G6_BM), chunk * BN,     \
                          (size_t)NE * N, (size_t)e * N, rowmap, use_map, rowscale, use_scale);                       \
  }
GEMM6_HD_INST(1)
GEMM6_HD_INST(2)
// (Q6_K experts: the dense kernel's body over tiles of at most 64 slots -- the engine builds the list for that size)
extern "C" __global__ __launch_bounds__(256, 2) void gemm__QTYPE14_ACT321_MOE_TILES1(
    const uint8_t* raw, const uint8_t* wh_unused, const signed char* aq, const float* asc, const short* absum, float* C,
    int M, int N, int K, int ldc, int accumulate, const int* tiles, const int* tstart, int e0, int e1, const int* rowmap,
    int use_map, const float* rowscale, int use_scale, int NE) {
  int ti, chunk;
  if (!moe_tile_of(tstart[e1] - tstart[e0], gridDim.x, ti, chunk)) return;
  ti += tstart[e0];
  const int e = tiles[1 + 3 * ti], r0 = tiles[2 + 3 * ti], nr = tiles[3 + 3 * ti];
  gemm6_body<true>(raw, aq, asc, C, M, N, K, ldc, 0, accumulate, 0, K >> 8, r0, min(nr, G6_BM), chunk * BN,
                   (size_t)NE * N, (size_t)e * N, rowmap, use_map, rowscale, use_scale);
}
