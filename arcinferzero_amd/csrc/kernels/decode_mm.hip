// "decode" module, part: gemv_mm, the matrix-vector form for 3..16 tokens on the matrix pipe (Q4_K, Q5_K, Q6_K, Q8_0,
// Q4_0, IQ4_NL, MXFP4, IQ4_XS, IQ3_S, Q3_K, IQ3_XXS).
//
// From a handful of tokens on, the dot-product GEMVs are bound by their vector ALU work (eight v_dot4 per token and
// 16-byte unit), not by memory, and past eight tokens the engine had only the prefill GEMM with its 64-token tiles.
// Here the int32 block sums come from v_mfma_i32_16x16x32_i8: a wave multiplies the 32 values of one block of 16
// weight rows with up to 16 tokens in one instruction, and the vector ALU is left with the f32 scale step of the
// prefill GEMM (reference zero/kernels/gemm.cl:439-488), for Q4_K and Q5_K
//   res += (sa[t][b] * (d[n] * sc[n][b])) * (float)I[t][n][b]  -  (sa[t][b] * (float)S[t][b]) * (dmin[n] * mn[n][b])
// with S the sum of the block's 32 int8 activations, for Q6_K (two int8 sub-scales per block, :457-464, 485)
//   res += d[n] * sa[t][b] * (float)(sc0[n][b] * I0[t][n][b] + sc1[n][b] * I1[t][n][b])
// and for Q8_0 (:445-447), Q4_0, IQ4_NL, MXFP4 and IQ4_XS (one scale per block)  res += (sa[t][b] * d[n][b]) * (float)I[t][n][b].  The
// weights are read once, as in the GEMVs.
//
// Tokens.  A work-group of 8 waves stages superblocks [s_begin, s_end) of the tokens in LDS -- int8 rows, and per block
// the 16 tokens' sa and (where the type has a min term) sa * S -- and keeps them for all its weight rows.  K in slices
// that fit LDS, one after the other inside the launch.
//
// Products.  Lane (n, g) = (lane % 16, lane / 16) is weight row n of a group of 16 rows as the instruction's column
// and supplies the 8 values 8 g .. 8 g + 7 of a block.  Q4_K / Q5_K: bytes 8 g .. 8 g + 7 of a 32-byte chunk of
// nibbles hold exactly those of the chunk's two blocks (low and high nibbles); Q5_K's fifth bits come from the word of
// the 16-byte unit those bytes lie in.  Q6_K: a block is the low or the high nibbles of 32 consecutive bytes of ql
// with two bits of 32 bytes of qh, and its two halves of 16 values have different scales: two instructions a block,
// the weights of the other half's lanes (g < 2, g >= 2) zeroed; the values enter as 4 (q - 32) (bit 5 flipped, the six
// bits at the top of the byte), the 4 goes into d.  Q8_0: the int8 values as they lie.  The instruction leaves the
// lane the sums of tokens 4 g .. 4 g + 3 with its row, whose scales it has decoded itself.  The min term of four
// blocks is one f32 matrix instruction (16 x 16 x 4) straight into the sums.
//
// Weights.  Were a lane to load the 8 bytes that the matrix instruction wants from it, an instruction would touch 16
// rows' lines for 32 bytes each: that form ran at 2 TB/s with or without its arithmetic.  Instead a lane loads 16
// bytes such that eight lanes (Q8_0: sixteen) cover one row's superblock in the type's main plane, several
// superblocks ahead in registers, and the wave turns a superblock's rows through a piece of LDS of its own into the
// matrix instruction's layout (LDS operations of one wave complete in order: no barrier).  Headers (Q6_K: the 16
// scales, Q8_0: the 8 block scales) come four superblocks at a time (lane (n, j): row n, superblock j of the four)
// through LDS in the same way, and so do the smaller planes (Q5_K's qh, Q6_K's qh and d), in whole lines.
//
// Work.  A work-group takes a contiguous run of 16-row groups (groups / gridDim.x of them, or one more); the run's
// (group, superblock) units, group-major, are cut into eight equal stretches, one per wave, so every wave streams the
// same amount whatever the number of groups.  A group that lies within one stretch is stored by its wave; one that is
// cut by a stretch boundary is added up after the work-group's one meeting, in wave order, by the wave in which it ends
// (it is that wave's first group).
#include "common.h"

#define MM_WAVES 8
#define MM_LDS_MAX (160 * 1024 - 1024)

typedef uint32_t mm_u2 __attribute__((ext_vector_type(2)));
typedef uint32_t mm_u4 __attribute__((ext_vector_type(4)));

// Per type: SB, the superblocks of a slice at most; QB, the bytes of a row's superblock in the main plane; D, the
// superblocks a wave has in flight; XB, the bytes per row and superblock of the second plane that goes through LDS in
// batches of four; MIN, whether the type has a min term; DPL, whether d is a plane of its own (2 bytes).
template <int QT> struct MmT;
template <> struct MmT<QT_Q4_K> { enum { SB = 24, QB = 128, D = 8, XB = 0, MIN = 1, DPL = 0 }; };
template <> struct MmT<QT_Q5_K> { enum { SB = 22, QB = 128, D = 4, XB = 32, MIN = 1, DPL = 0 }; };
// (Q6_K: two -- with four the kernel needed 270 registers and kept 14 of them in scratch memory, 60 bytes a lane written
//  and read back per superblock: 8 tokens at 17408 x 5120 31.1 -> 24.5 us)
template <> struct MmT<QT_Q6_K> { enum { SB = 20, QB = 128, D = 2, XB = 64, MIN = 0, DPL = 1 }; };
template <> struct MmT<QT_Q8_0> { enum { SB = 24, QB = 256, D = 4, XB = 0, MIN = 0, DPL = 0 }; };
template <> struct MmT<QT_Q4_0> { enum { SB = 24, QB = 128, D = 8, XB = 0, MIN = 0, DPL = 0 }; };
template <> struct MmT<QT_IQ4_NL> : MmT<QT_Q4_0> {};
template <> struct MmT<QT_MXFP4> : MmT<QT_Q4_0> {};
template <> struct MmT<QT_IQ4_XS> { enum { SB = 24, QB = 128, D = 8, XB = 0, MIN = 0, DPL = 0 }; };
// (IQ3_S: the main plane is the 8 index bytes per block, the second the sign bits, the header the ninth bits and scale
//  nibbles, 12 bytes; the codebook, 2 KiB, sits behind the groups' sums in LDS)
template <> struct MmT<QT_IQ3_S> { enum { SB = 22, QB = 64, D = 8, XB = 32, MIN = 0, DPL = 1 }; };
// (Q3_K: planes of the same sizes -- 8 bytes of bit pairs per block, the words of third bits, 12 bytes of scales)
template <> struct MmT<QT_Q3_K> : MmT<QT_IQ3_S> {};
// (IQ3_XXS: the index bytes and the blocks' words of sign codes and scales likewise; no header plane)
template <> struct MmT<QT_IQ3_XXS> : MmT<QT_IQ3_S> {};
// LDS: per superblock of a slice 4096 bytes of tokens and 512 of sa (512 more of sa * S); per wave the main plane's rows
// of one superblock, 1 KiB of headers, the second plane's four superblocks, 256 bytes of d; then 1 KiB per group whose
// sums wait for the last slice (as many as fit, 12 at most)
template <int QT> struct MmL {
  static constexpr int TOK = 4096 + 512 + (MmT<QT>::MIN ? 512 : 0);
  static constexpr int WQ = MmT<QT>::QB * 16 < 2048 ? 2048 : MmT<QT>::QB * 16;  // (also the wave's two partial sums: 2 KiB)
  static constexpr int WH = 1024, WX = MmT<QT>::XB * 64, WD = MmT<QT>::DPL ? 256 : 0;
  static constexpr int GRID = QT == QT_IQ3_S ? 2048 : QT == QT_IQ3_XXS ? 1024 : 0;
  static constexpr int WSZ = WQ + WH + WX + WD;
  static constexpr int FREE = (MM_LDS_MAX - MmT<QT>::SB * TOK - MM_WAVES * WSZ - GRID) / 1024;
  static constexpr int GA = FREE < 12 ? FREE : 12;
  static constexpr int OGRID = MmT<QT>::SB * TOK + MM_WAVES * WSZ + GA * 1024;
  static constexpr int LDS = OGRID + GRID;
  static_assert(GA >= 1, "no room for the groups' sums");
};

template <int QT> struct MmQ { mm_u4 r[MmT<QT>::QB / 64]; };  // the lane's 16-byte pieces of a superblock of 16 rows
template <int QT> struct MmX { mm_u4 r[MmT<QT>::XB / 16 > 0 ? MmT<QT>::XB / 16 : 1]; uint32_t d; };  // of four superblocks' second plane
// a superblock as the products take it: the lane's 8 bytes of each 32-byte chunk of the main plane, the header
// (Q4_0, IQ4_NL, MXFP4 and IQ4_XS: of each 16-byte block)
// (IQ3_S: c[b].x the lane's two index bytes of block b, sg the row's eight words of sign bits)
template <int QT> struct MmSb {
  mm_u2 c[qt_nib16(QT) || QT == QT_IQ4_XS || QT == QT_IQ3_S || QT == QT_Q3_K || QT == QT_IQ3_XXS ? 8 : MmT<QT>::QB / 32];
  mm_u4 h;
  mm_u2 x[2];
  uint32_t d;
  mm_u4 sg[QT == QT_IQ3_S || QT == QT_Q3_K || QT == QT_IQ3_XXS ? 2 : 1];
};

// one slice of K, superblocks [s_begin, s_end): at most MmT<QT>::SB of them
template <int QT>
__device__ inline void mm_slice(uint8_t* lds, const uint8_t* __restrict__ raw, int N, int K,
                                const signed char* __restrict__ aq, const float* __restrict__ asc,
                                const short* __restrict__ absum, int M, int T, float* C, int ldc, int c_off, int accumulate,
                                int s_begin, int s_end, float* GA, bool first, bool last) {
  using TT = MmT<QT>;
  using LL = MmL<QT>;
  constexpr int QB = TT::QB, NQ = QB / 64, D = TT::D, LPRW = QB / 16, RPI = 64 / LPRW;
  constexpr bool Q45 = QT == QT_Q4_K || QT == QT_Q5_K;
  constexpr bool B16 = qt_nib16(QT) || QT == QT_IQ4_XS;  // a block is 16 bytes: low nibbles values 0..15, high 16..31
  constexpr int HB = QT == QT_IQ3_XXS ? 0 : QT == QT_IQ4_XS || QT == QT_MXFP4 ? 8 : QT == QT_IQ3_S || QT == QT_Q3_K ? 12 : 16;  // bytes of a row's superblock in the header plane
  constexpr bool I3 = QT == QT_IQ3_S || QT == QT_Q3_K || QT == QT_IQ3_XXS;  // (the types of these plane sizes)
  constexpr bool K3 = QT == QT_Q3_K, X3 = QT == QT_IQ3_XXS;
  const int tid = threadIdx.x, lane = tid & 63, n16 = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (a scalar: what follows from it is scalar arithmetic)
  const int nsb = K >> 8, sbs = s_end - s_begin, Ks = sbs * 256, nb = sbs * 8;
  uint8_t* A = lds;                            // [16][Ks] int8; 16-byte piece k of token t sits at piece k ^ t of its row
  float* SA = (float*)(lds + 16 * Ks);         // [nb][16] sa
  float* U = SA + nb * 16;                     // [nb][16] sa * S (types with a min term)
  uint8_t* WB = (uint8_t*)(SA + (TT::MIN ? 2 : 1) * nb * 16);  // per wave: WQ, WH, WX, WD
  uint8_t* WQ = WB + wave * LL::WSZ;
  uint8_t* WH = WQ + LL::WQ;
  uint8_t* WX = WH + LL::WH;
  uint8_t* WD = WX + LL::WX;
  // the planes (all have the main plane first, a row's superblocks together)
  size_t o_hdr, o_x = 0, o_d = 0;
  if constexpr (Q45) {
    const PlanesQ4K pl = planes_q4k((size_t)N, nsb);
    o_hdr = pl.hdr; o_x = pl.qh;
  } else if constexpr (QT == QT_Q6_K) {
    const PlanesQ6K pl = planes_q6k((size_t)N, nsb);
    o_hdr = pl.sc; o_x = pl.qh; o_d = pl.d;
  } else if constexpr (QT == QT_Q8_0) {
    o_hdr = planes_q80((size_t)N, nsb).d;
  } else if constexpr (qt_nib16(QT)) {
    o_hdr = planes_q40((size_t)N, nsb).d;  // (MXFP4: its scale bytes, at the same place)
  } else if constexpr (X3) {
    const PlanesIQ3XXS pl = planes_iq3xxs((size_t)N, nsb);
    o_hdr = 0; o_x = pl.ss; o_d = pl.d;  // (no header plane)
  } else if constexpr (I3) {
    const PlanesIQ3S pl = planes_iq3s((size_t)N, nsb);
    o_hdr = pl.hd; o_x = pl.sg; o_d = pl.d;
  } else {
    o_hdr = planes_iq4xs((size_t)N, nsb).hdr;
  }
  const uint8_t* qs = raw;
  const uint8_t* hd = raw + o_hdr;
  const uint8_t* xp = raw + o_x;
  const uint8_t* dp = raw + o_d;
  const int groups = (N + 15) >> 4, gd = (int)gridDim.x;
  const int gb0 = (int)((long)blockIdx.x * groups / gd), gb1 = (int)((long)(blockIdx.x + 1) * groups / gd);
  const int units = (gb1 - gb0) * sbs;         // >= 1: the grid has at most `groups` work-groups
  const int u0 = wave * units / MM_WAVES, u1 = (wave + 1) * units / MM_WAVES;
  const int ulast = max(u1 - 1, 0);            // (a wave without units loads unit 0 and drops it)
  // unit -> group of the run (units below 2^27): the high word of u * ceil(2^32 / sbs)
  const uint32_t magic = 0xFFFFFFFFu / (uint32_t)sbs + 1u;
  auto group_of = [&](int u) { return sbs == 1 ? u : (int)__umulhi((uint32_t)u, magic); };

  // (the unit's base is a scalar; a lane adds its row of the group -- rows past the matrix: the last -- times the row
  //  stride, below 2^24, and its piece)
  const uint32_t row_stride = (uint32_t)nsb * QB, piece_off = (uint32_t)(lane % LPRW) * 16;
  auto qload = [&](MmQ<QT>& q, int u) {  // u: the same in the whole wave, within the run
    const int gl = group_of(u), sb = u - gl * sbs;
    const int g0 = (gb0 + gl) * 16;
    const uint8_t* base = qs + ((size_t)g0 * nsb + (s_begin + sb)) * QB;
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
      const uint32_t rel = (uint32_t)min(i * RPI + lane / LPRW, N - 1 - g0);
      // (the main plane is read once per launch: non-temporal, so that the caches keep the tokens and the small planes
      //  -- 8 tokens, us: Q4_K 17408 x 5120 21.1 -> 20.5, 151936 x 5120 100 -> 96, Q8_0 155 -> 139)
      q.r[i] = __builtin_nontemporal_load((const mm_u4*)(base + (__umul24(rel, row_stride) + piece_off)));
    }
  };
  auto hload = [&](mm_u4& h, int ub) {  // the headers of units ub .. ub + 3 (past the stretch: its last)
    const int u = min(ub + g, ulast);
    const int gl = group_of(u), sb = u - gl * sbs;
    const int r = min((gb0 + gl) * 16 + n16, N - 1);
    if constexpr (HB == 0) {
      h = mm_u4{0u, 0u, 0u, 0u};
    } else if constexpr (HB == 16) {
      h = *(const mm_u4*)(hd + ((size_t)r * nsb + s_begin + sb) * 16);
    } else if constexpr (HB == 12) {
      const uint32_t* hp = (const uint32_t*)(hd + ((size_t)r * nsb + s_begin + sb) * 12);
      h = mm_u4{hp[0], hp[1], hp[2], 0};
    } else {
      const mm_u2 h2 = *(const mm_u2*)(hd + ((size_t)r * nsb + s_begin + sb) * 8);
      h = mm_u4{h2.x, h2.y, 0, 0};
    }
  };
  // the second plane of units ub .. ub + 3: a row's XB bytes of a unit are XB / 16 lanes' pieces, whole lines where the
  // four units are superblocks of one group; Q6_K's d with the header's lanes
  auto xload = [&](MmX<QT>& x, int ub) {
    if constexpr (TT::XB > 0) {
      constexpr int PU = TT::XB / 16, RX = 64 / (4 * PU);  // pieces per unit and row; rows per instruction
#pragma unroll
      for (int i = 0; i < PU; ++i) {
        const int row = i * RX + lane / (4 * PU), j = (lane % (4 * PU)) / PU, p = lane % PU;
        const int u = min(ub + j, ulast);
        const int gl = group_of(u), sb = u - gl * sbs;
        const int r = min((gb0 + gl) * 16 + row, N - 1);
        x.r[i] = *(const mm_u4*)(xp + ((size_t)r * nsb + s_begin + sb) * TT::XB + p * 16);
      }
    }
    if constexpr (TT::DPL) {
      const int u = min(ub + g, ulast);
      const int gl = group_of(u), sb = u - gl * sbs;
      const int r = min((gb0 + gl) * 16 + n16, N - 1);
      x.d = *(const unsigned short*)(dp + ((size_t)r * nsb + s_begin + sb) * 2);
    }
  };

  // ---- staging.  Loads first: the tokens' int8 rows (wave w: rows 2 w and 2 w + 1, 16-byte pieces lane, lane + 64, ..),
  // their scales and sums (asc [K / 32][M], absum [K / 16][M]), then the wave's first superblocks right behind them:
  // loads come back in order, so the stores below wait for the tokens alone while the weights are on their way.
  constexpr int NCH = (TT::SB * 16 + 63) / 64;  // pieces per lane and row at most
  constexpr int NSC = (TT::SB * 8 * 16 + 511) / 512;  // (block, token) pairs per thread at most
  const int cpr = Ks >> 4;
  mm_u4 va[2][NCH];
  float vs[NSC];
  int vu[NSC];
#pragma unroll
  for (int r2 = 0; r2 < 2; ++r2) {
    const int t = 2 * wave + r2, tt = t < T ? t : 0;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int k16 = min(lane + 64 * i, cpr - 1);
      va[r2][i] = *(const mm_u4*)(aq + (size_t)tt * K + (size_t)s_begin * 256 + k16 * 16);
    }
  }
#pragma unroll
  for (int i = 0; i < NSC; ++i) {
    const int idx = min(tid + 512 * i, nb * 16 - 1), b = s_begin * 8 + (idx >> 4), t = idx & 15, tt = t < T ? t : 0;
    vs[i] = asc[(size_t)b * M + tt];
    if constexpr (TT::MIN) vu[i] = (int)absum[(size_t)(2 * b) * M + tt] + (int)absum[(size_t)(2 * b + 1) * M + tt];
  }
  __builtin_amdgcn_sched_barrier(0);
  MmQ<QT> q[D];
  MmX<QT> xq;
  mm_u4 hq0, hq1;
  hload(hq0, u0);
  hload(hq1, u0 + 4);
  xload(xq, u0);
#pragma unroll
  for (int k = 0; k < D; ++k) qload(q[k], min(u0 + k, ulast));
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r2 = 0; r2 < 2; ++r2) {
    const int t = 2 * wave + r2;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int k16 = min(lane + 64 * i, cpr - 1);  // (clamped lanes store the same bytes again)
      mm_u4 v = va[r2][i];
      if (t >= T) v = mm_u4{0, 0, 0, 0};
      *(mm_u4*)(A + t * Ks + ((k16 ^ t) << 4)) = v;
    }
  }
#pragma unroll
  for (int i = 0; i < NSC; ++i) {
    const int idx = min(tid + 512 * i, nb * 16 - 1), t = idx & 15;
    const float sa = t < T ? vs[i] : 0.0f;
    SA[idx] = sa;
    if constexpr (TT::MIN) U[idx] = sa * (float)vu[i];
  }
  __syncthreads();

  // the lane's places in the wave's LDS.  Main plane: piece p of row r of a superblock at 16-byte slot 16 p + (r ^ 2 p)
  // (Q8_0, 16 pieces a row: 16 p + (r ^ p)), so that the writes (a quarter wave: two rows' eight pieces, or one row's
  // sixteen) and the reads (half a wave: one piece of 16 rows, 8 bytes a lane) each go to all banks once
  int wq[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int p = lane % LPRW, r = i * RPI + lane / LPRW;
    wq[i] = I3 ? r * 64 + ((p ^ (r >> 2)) << 4) : (16 * p + (r ^ (LPRW == 8 ? 2 * p : p))) << 4;
  }
  // (the lane's 8 bytes: bytes 8 g .. of each 32-byte chunk; for the 16-byte blocks bytes 8 (g & 1) .. of each block,
  //  whose low nibbles are the values of lanes g < 2 and whose high nibbles those of g >= 2)
  // (IQ3_S: the row's 64 index bytes lie together, 16-byte pieces XOR-ed with row / 4; the lane's are bytes 8 b + 2 g, + 1)
  constexpr int NC = B16 || I3 ? 8 : QB / 32;
  int rd[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int p = B16 ? c : 2 * c + (g >> 1);
    rd[c] = K3 ? n16 * 64 + (((c >> 1) ^ (n16 >> 2)) << 4) + 8 * (c & 1) + 4 * (g >> 1)  // (Q3_K: the word of the lane's half)
            : I3 ? n16 * 64 + (((c >> 1) ^ (n16 >> 2)) << 4) + 8 * (c & 1) + 2 * g
               : ((16 * p + (n16 ^ (LPRW == 8 ? 2 * p : p))) << 4) + (g & 1) * 8;
  }
  const uint8_t* arow = A + n16 * Ks + (g & 1) * 8;

  // the products of one superblock (sbk: its index within the slice) of the lane's row, into acc
  auto products = [&](const MmSb<QT>& h, int sbk, v4f& acc) {
    const int b0 = sbk * 8;
    long av[8];
    float4 sa4[8];
    // the tokens' values and scales of the superblock's blocks (Q6_K: of four blocks at a time, for the registers)
    auto tokens = [&](int from, int to) {
#pragma unroll
      for (int b = from; b < to; ++b) {
        av[b] = *(const long*)(arow + ((sbk * 16 + ((2 * b + (g >> 1)) ^ n16)) << 4));
        sa4[b] = *(const float4*)(SA + (b0 + b) * 16 + 4 * g);
      }
    };
    if constexpr (QT != QT_Q6_K) tokens(0, 8);
    if constexpr (Q45) {
      const float d = f16_bits_to_f32(h.h.x), dmin = f16_bits_to_f32(h.h.x >> 16);
      const float ua = U[(b0 + g) * 16 + n16], ub = U[(b0 + 4 + g) * 16 + n16];
      int sc[8], mn[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) q4k_scales_pair(h.h.y, h.h.z, h.h.w, j, sc[2 * j], sc[2 * j + 1], mn[2 * j], mn[2 * j + 1]);
      v4i I[8];
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const mm_u2 cw = h.c[b >> 1];
        uint32_t w0 = ((b & 1) ? cw.x >> 4 : cw.x) & 0x0F0F0F0Fu, w1 = ((b & 1) ? cw.y >> 4 : cw.y) & 0x0F0F0F0Fu;
        if constexpr (QT == QT_Q5_K) {
          // the fifth bits: word H of the 16-byte unit the lane's 8 bytes lie in (unit 2 c + g / 2 of the superblock),
          // whose bits 4 + k and k belong to the low and the high nibbles of the unit's word k; the lane's are words
          // 2 (g & 1) and 2 (g & 1) + 1
          const uint32_t H = (b >> 1) < 2 ? ((b >> 1) == 0 ? h.x[0].x : h.x[0].y) : ((b >> 1) == 2 ? h.x[1].x : h.x[1].y);
          const int k0 = 2 * (g & 1);
          if (b & 1) {
            w0 |= (H << (4 - k0)) & 0x10101010u;
            w1 |= (H << (3 - k0)) & 0x10101010u;
          } else {
            w0 |= (H >> k0) & 0x10101010u;
            w1 |= (H >> (k0 + 1)) & 0x10101010u;
          }
        }
        const long wv = (long)(((unsigned long)w1 << 32) | w0);
        v4i z = {0, 0, 0, 0};
        I[b] = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wv, z, 0, 0, 0);
      }
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const float ws = d * (float)sc[b];
        acc[0] = fmaf((float)I[b][0], sa4[b].x * ws, acc[0]);
        acc[1] = fmaf((float)I[b][1], sa4[b].y * ws, acc[1]);
        acc[2] = fmaf((float)I[b][2], sa4[b].z * ws, acc[2]);
        acc[3] = fmaf((float)I[b][3], sa4[b].w * ws, acc[3]);
      }
      // the min term of each half's four blocks, - sum_b (sa S)[t][b] (dmin mn)[n][b], as one f32 matrix instruction
      const int m0 = g == 0 ? mn[0] : g == 1 ? mn[1] : g == 2 ? mn[2] : mn[3];
      const int m1 = g == 0 ? mn[4] : g == 1 ? mn[5] : g == 2 ? mn[6] : mn[7];
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ua, -(dmin * (float)m0), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ub, -(dmin * (float)m1), acc, 0, 0, 0);
    } else if constexpr (QT == QT_Q6_K) {
      // block b = 4 n2 + hb of the superblock: the low (hb < 2) or high nibbles of ql bytes 64 n2 + 32 (hb & 1) + 0..31
      // (chunk 2 n2 + (hb & 1)) with bits 2 hb, 2 hb + 1 of qh bytes 32 n2 + 0..31; scales 2 b and 2 b + 1 for its
      // halves, which are the lanes g < 2 and g >= 2
      const uint32_t keep_a = g < 2 ? 0xFCFCFCFCu : 0u, keep_b = g < 2 ? 0u : 0xFCFCFCFCu;
      const float d = 0.25f * f16_bits_to_f32(h.d);
      v4f part = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        if ((b & 3) == 0) {
          __builtin_amdgcn_sched_barrier(0);
          tokens(b, b + 4);
        }
        const int n2 = b >> 2, hb = b & 3;
        const mm_u2 L = h.c[2 * n2 + (hb & 1)], H = h.x[n2];
        uint32_t w[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const uint32_t l = k ? L.y : L.x, hh = k ? H.y : H.x;
          const uint32_t nib = hb < 2 ? l << 2 : l >> 2;                         // the nibble at bits 2..5
          const uint32_t top = hb == 3 ? hh : hh << (6 - 2 * hb);                // the two high bits at 6..7
          w[k] = (((nib & 0x3C3C3C3Cu) | (top & 0xC0C0C0C0u)) ^ 0x80808080u);   // 4 (q - 32) as int8
        }
        const long wa = (long)(((unsigned long)(w[1] & keep_a) << 32) | (w[0] & keep_a));
        const long wb = (long)(((unsigned long)(w[1] & keep_b) << 32) | (w[0] & keep_b));
        v4i z = {0, 0, 0, 0};
        const v4i Ia = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wa, z, 0, 0, 0);
        const v4i Ib = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wb, z, 0, 0, 0);
        const uint32_t sw = b < 2 ? h.h.x : b < 4 ? h.h.y : b < 6 ? h.h.z : h.h.w;
        // (the sums are below 2^23 in size -- 16 x 127 x 128 -- and the scales int8: 24-bit multiplies)
        const int sca = (int)(signed char)(sw >> (16 * (b & 1))), scb = (int)(signed char)(sw >> (16 * (b & 1) + 8));
        part[0] = fmaf((float)(__mul24(sca, Ia[0]) + __mul24(scb, Ib[0])), sa4[b].x, part[0]);
        part[1] = fmaf((float)(__mul24(sca, Ia[1]) + __mul24(scb, Ib[1])), sa4[b].y, part[1]);
        part[2] = fmaf((float)(__mul24(sca, Ia[2]) + __mul24(scb, Ib[2])), sa4[b].z, part[2]);
        part[3] = fmaf((float)(__mul24(sca, Ia[3]) + __mul24(scb, Ib[3])), sa4[b].w, part[3]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(d, part[i], acc[i]);
    } else if constexpr (X3) {
      // block b: indices 2 g and 2 g + 1 of its eight (a byte each) name codebook words of four magnitudes; the signs of
      // the lane's eight values are the block's sign code g, the scale the top nibble of that word; d / 4
      // (reference src/quants.h:220-239, zero/kernels/decode.cl:183-478)
      const uint32_t* grid = (const uint32_t*)(lds + LL::OGRID);
      const float d3 = 0.25f * f16_bits_to_f32(h.d);
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const uint32_t q16 = h.c[b].x;
        const uint32_t a = b < 4 ? h.sg[0][b & 3] : h.sg[1][b & 3];
        const uint32_t s8 = iq3xxs_signs8(a, g);
        const uint32_t w0 = iq3s_signed4(grid[q16 & 0xFFu], s8 & 0xFu), w1 = iq3s_signed4(grid[(q16 >> 8) & 0xFFu], s8 >> 4);
        const long wv = (long)(((unsigned long)w1 << 32) | w0);
        v4i z = {0, 0, 0, 0};
        const v4i I = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wv, z, 0, 0, 0);
        const float d = d3 * (float)(1 + 2 * (int)(a >> 28));
        acc[0] = fmaf((float)I[0], sa4[b].x * d, acc[0]);
        acc[1] = fmaf((float)I[1], sa4[b].y * d, acc[1]);
        acc[2] = fmaf((float)I[2], sa4[b].z * d, acc[2]);
        acc[3] = fmaf((float)I[3], sa4[b].w * d, acc[3]);
      }
    } else if constexpr (K3) {
      // block b: the lane's eight values 8 g .. 8 g + 7 are the fields 2 g and 2 g + 1 of the block's bit words; the
      // block's two 16-value halves have a scale each, so, as for Q6_K, two products with the other half's lanes zeroed
      // (values 0..15 are the lanes g < 2) and sc0 * I0 + sc1 * I1 in integers (zero/kernels/decode.cl:203-222)
      const float d3 = f16_bits_to_f32(h.d);
      v4f part = {0.0f, 0.0f, 0.0f, 0.0f};
      const uint32_t keep0 = g < 2 ? 0xFFFFFFFFu : 0u, keep1 = ~keep0;
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const uint32_t D = h.c[b].x;
        const uint32_t H = b < 4 ? h.sg[0][b & 3] : h.sg[1][b & 3];
        const uint32_t w0 = q3k_vals(D, H, 2 * g), w1 = q3k_vals(D, H, 2 * g + 1);
        const long wa = (long)(((unsigned long)(w1 & keep0) << 32) | (w0 & keep0));
        const long wb = (long)(((unsigned long)(w1 & keep1) << 32) | (w0 & keep1));
        v4i z = {0, 0, 0, 0};
        const v4i Ia = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wa, z, 0, 0, 0);
        const v4i Ib = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wb, z, 0, 0, 0);
        int sca, scb;
        q3k_scales(h.h.x, h.h.y, h.h.z, b, sca, scb);
        part[0] = fmaf((float)(__mul24(sca, Ia[0]) + __mul24(scb, Ib[0])), sa4[b].x, part[0]);
        part[1] = fmaf((float)(__mul24(sca, Ia[1]) + __mul24(scb, Ib[1])), sa4[b].y, part[1]);
        part[2] = fmaf((float)(__mul24(sca, Ia[2]) + __mul24(scb, Ib[2])), sa4[b].z, part[2]);
        part[3] = fmaf((float)(__mul24(sca, Ia[3]) + __mul24(scb, Ib[3])), sa4[b].w, part[3]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(d3, part[i], acc[i]);
    } else if constexpr (I3) {
      // block b: indices 2 g and 2 g + 1 of its eight (a byte each and a ninth bit from byte b of the header) name
      // codebook words of four magnitudes, the signs are bits 8 g .. 8 g + 7 of the block's word; scale 1 + 2 x nibble b
      // of the header's third word, times d (reference src/quants.h IQ3_S, zero/kernels/decode.cl:183-478)
      const uint32_t* grid = (const uint32_t*)(lds + LL::OGRID);
      const float d3 = f16_bits_to_f32(h.d);
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const uint32_t q16 = h.c[b].x;
        const uint32_t n9 = (b < 4 ? h.h.x : h.h.y) >> (8 * (b & 3) + 2 * g);
        const uint32_t g0 = grid[(q16 & 0xFFu) | ((n9 & 1u) << 8)], g1 = grid[((q16 >> 8) & 0xFFu) | ((n9 & 2u) << 7)];
        const uint32_t sw = b < 4 ? h.sg[0][b & 3] : h.sg[1][b & 3];
        const uint32_t s8 = sw >> (8 * g);
        const uint32_t w0 = iq3s_signed4(g0, s8 & 0xFu), w1 = iq3s_signed4(g1, (s8 >> 4) & 0xFu);
        const long wv = (long)(((unsigned long)w1 << 32) | w0);
        v4i z = {0, 0, 0, 0};
        const v4i I = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wv, z, 0, 0, 0);
        const float d = d3 * (float)(1 + 2 * (int)((h.h.z >> (4 * b)) & 0xFu));
        acc[0] = fmaf((float)I[0], sa4[b].x * d, acc[0]);
        acc[1] = fmaf((float)I[1], sa4[b].y * d, acc[1]);
        acc[2] = fmaf((float)I[2], sa4[b].z * d, acc[2]);
        acc[3] = fmaf((float)I[3], sa4[b].w * d, acc[3]);
      }
    } else if constexpr (B16) {
      // block b is the 16 bytes 16 b .. of the row's 128; Q4_0: value nibble - 8, f16 scale entry b of the header (IQ4_NL:
      // the table's value; MXFP4: its table's, and a scale byte);
      // IQ4_XS: the table's value of the nibble, d in the header's first half word and a 6-bit scale - 32 per block (low
      // four bits in the second word, high two in the upper half of the first)
      const int sh = 4 * (g >> 1);
      const float d4 = f16_bits_to_f32(h.h.x);
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const mm_u2 cw = h.c[b];
        uint32_t w0, w1;
        float d;
        if constexpr (QT == QT_MXFP4) {  // (the header: the eight blocks' scale bytes)
          w0 = mxfp4_lookup(cw.x >> sh);
          w1 = mxfp4_lookup(cw.y >> sh);
          d = e8m0_half((b < 4 ? h.h.x : h.h.y) >> (8 * (b & 3)));
        } else if constexpr (qt_nib16(QT)) {
          w0 = nib_vals<QT>(cw.x >> sh);
          w1 = nib_vals<QT>(cw.y >> sh);
          const uint32_t dw = b < 2 ? h.h.x : b < 4 ? h.h.y : b < 6 ? h.h.z : h.h.w;
          d = f16_bits_to_f32((b & 1) ? dw >> 16 : dw);
        } else {
          w0 = iq4_lookup(cw.x >> sh);
          w1 = iq4_lookup(cw.y >> sh);
          const int ls = (int)(((h.h.y >> (4 * b)) & 0xFu) | ((((h.h.x >> 16) >> (2 * b)) & 3u) << 4)) - 32;
          d = d4 * (float)ls;
        }
        const long wv = (long)(((unsigned long)w1 << 32) | w0);
        v4i z = {0, 0, 0, 0};
        const v4i I = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wv, z, 0, 0, 0);
        acc[0] = fmaf((float)I[0], sa4[b].x * d, acc[0]);
        acc[1] = fmaf((float)I[1], sa4[b].y * d, acc[1]);
        acc[2] = fmaf((float)I[2], sa4[b].z * d, acc[2]);
        acc[3] = fmaf((float)I[3], sa4[b].w * d, acc[3]);
      }
    } else {
      // Q8_0: block b is bytes 32 b .. 32 b + 31 of the row's 256, its f16 scale entry b of the 16-byte header
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const mm_u2 cw = h.c[b];
        const long wv = (long)(((unsigned long)cw.y << 32) | cw.x);
        v4i z = {0, 0, 0, 0};
        const v4i I = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wv, z, 0, 0, 0);
        const uint32_t dw = b < 2 ? h.h.x : b < 4 ? h.h.y : b < 6 ? h.h.z : h.h.w;
        const float d = f16_bits_to_f32((b & 1) ? dw >> 16 : dw);
        acc[0] = fmaf((float)I[0], sa4[b].x * d, acc[0]);
        acc[1] = fmaf((float)I[1], sa4[b].y * d, acc[1]);
        acc[2] = fmaf((float)I[2], sa4[b].z * d, acc[2]);
        acc[3] = fmaf((float)I[3], sa4[b].w * d, acc[3]);
      }
    }
  };

  // lane (n16, g) holds tokens 4 g .. 4 g + 3 of row n16 of a group
  const int tmax = T > 8 ? 16 : T;  // (9-16 tokens: the chunk has 16 rows, those from T on come out as zeros)
  // GA: the work-group's groups' sums over the slices so far, in LDS ([group][16 tokens][16 rows]; a load from C at
  // every group's end would wait for all the weights in flight behind it): C is written by the last slice alone
  auto store = [&](v4f v, int gl) {
    const int n = (gb0 + gl) * 16 + n16;
    if (GA) {
      float* ga = GA + gl * 256 + 64 * g + n16;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (!first) v[i] += ga[16 * i];
        if (!last) ga[16 * i] = v[i];
      }
      if (!last) return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 4 * g + i;
      if (t < tmax && n < N) {
        float* cp = C + (size_t)t * ldc + c_off + n;
        *cp = accumulate ? *cp + v[i] : v[i];
      }
    }
  };

  const int gf = group_of(min(u0, ulast));  // the stretch's first group
  v4f acc = {0.0f, 0.0f, 0.0f, 0.0f}, ph = acc, pt = acc;  // running sums; the cut group at the head, at the tail
  // unit u: its rows out of qq through the wave's LDS, qq refilled with the unit D on (past the stretch the last unit
  // again: the same loads on every path), the products
  auto sbstep = [&](MmQ<QT>& qq, int u, int j) {
    if (u < u1) {
#pragma unroll
      for (int i = 0; i < NQ; ++i) *(mm_u4*)(WQ + wq[i]) = qq.r[i];
    }
    qload(qq, min(u + D, ulast));
    if (u < u1) {
      MmSb<QT> s;
      if constexpr (I3) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
          s.c[c] = mm_u2{K3 ? *(const uint32_t*)(WQ + rd[c]) : (uint32_t) * (const unsigned short*)(WQ + rd[c]), 0u};
        s.sg[0] = *(const mm_u4*)(WX + (j * 16 + n16) * 32);
        s.sg[1] = *(const mm_u4*)(WX + (j * 16 + n16) * 32 + 16);
        s.d = *(const uint32_t*)(WD + ((j * 16 + n16) << 2));
      } else {
#pragma unroll
        for (int c = 0; c < NC; ++c) s.c[c] = *(const mm_u2*)(WQ + rd[c]);
      }
      s.h = *(const mm_u4*)(WH + ((j * 16 + n16) << 4));
      if constexpr (QT == QT_Q5_K) {
        // words g / 2, 2 + g / 2, 4 + g / 2, 6 + g / 2 of the row's 8 words of fifth bits
        const uint8_t* xr = WX + (j * 16 + n16) * 32 + 4 * (g >> 1);
        s.x[0].x = *(const uint32_t*)(xr);
        s.x[0].y = *(const uint32_t*)(xr + 8);
        s.x[1].x = *(const uint32_t*)(xr + 16);
        s.x[1].y = *(const uint32_t*)(xr + 24);
      }
      if constexpr (QT == QT_Q6_K) {
        // bytes 32 n2 + 8 g .. + 7 of the row's 64 bytes of qh (16-byte pieces XOR-ed with r / 4 against conflicts)
        const uint8_t* xr = WX + (j * 16 + n16) * 64 + (g & 1) * 8;
        s.x[0] = *(const mm_u2*)(xr + ((((g >> 1)) ^ (n16 >> 2)) << 4));
        s.x[1] = *(const mm_u2*)(xr + (((2 + (g >> 1)) ^ (n16 >> 2)) << 4));
        s.d = *(const uint32_t*)(WD + ((j * 16 + n16) << 2));
      }
      const int gl = group_of(u), sb = u - gl * sbs;
      products(s, sb, acc);
      if (sb == sbs - 1 || u == u1 - 1) {  // the group ends here, or the stretch does
        if (gl * sbs >= u0 && (gl + 1) * sbs <= u1) store(acc, gl);
        else if (gl == gf) ph = acc;
        else pt = acc;
        acc = v4f{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
  };
  // a batch of four units' headers (and second plane) into the wave's LDS, the next ones asked for
  auto batch = [&](mm_u4& hq, int ub_next_h, int ub_next_x) {
    *(mm_u4*)(WH + ((g * 16 + n16) << 4)) = hq;
    hload(hq, ub_next_h);
    if constexpr (TT::XB > 0) {
      constexpr int PU = TT::XB / 16, RX = 64 / (4 * PU);
#pragma unroll
      for (int i = 0; i < PU; ++i) {
        const int row = i * RX + lane / (4 * PU), j = (lane % (4 * PU)) / PU, p = lane % PU;
        const int pp = QT == QT_Q6_K ? p ^ (row >> 2) : p;
        *(mm_u4*)(WX + (j * 16 + row) * TT::XB + pp * 16) = xq.r[i];
      }
    }
    if constexpr (TT::DPL) *(uint32_t*)(WD + ((g * 16 + n16) << 2)) = xq.d;
    if constexpr (TT::XB > 0 || TT::DPL) xload(xq, ub_next_x);
  };
#pragma unroll 1
  for (int u = u0; u < u1; u += 8) {
    batch(hq0, u + 8, u + 4);
#pragma unroll
    for (int k = 0; k < 4; ++k) sbstep(q[k % D], u + k, k);
    batch(hq1, u + 12, u + 8);
#pragma unroll
    for (int k = 4; k < 8; ++k) sbstep(q[k % D], u + k, k - 4);
  }

  // the cut groups: the partial sums into the wave's own LDS (two slots of [16 tokens][16 rows]), one meeting, then the
  // wave in which a cut group ends -- it is that wave's first -- adds its parts in wave order
  float* part = (float*)WQ;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    part[(4 * g + i) * 16 + n16] = ph[i];
    part[256 + (4 * g + i) * 16 + n16] = pt[i];
  }
  __syncthreads();
  if (u1 > u0 && gf * sbs < u0 && (gf + 1) * sbs <= u1) {
    v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int w = 0; w <= wave; ++w) {
      const int a0 = w * units / MM_WAVES, a1 = (w + 1) * units / MM_WAVES;
      if (a1 > a0 && a1 > gf * sbs && a0 < (gf + 1) * sbs) {
        const float* pw = (const float*)(WB + w * LL::WSZ) + (group_of(a0) == gf ? 0 : 256);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += pw[(4 * g + i) * 16 + n16];
      }
    }
    store(v, gf);
  }
}

// Superblocks [s_begin, s_end) of K, in slices that the work-group takes one after the other.  With more than one slice
// the sums of a work-group's groups wait in LDS for the last slice (as many groups as the type's LDS leaves room for);
// with more groups than that a later slice adds to what the work-group itself has stored in C (other waves of it, as
// the stretches fall: the meetings between the slices order those stores and loads within the work-group).
template <int QT>
__device__ inline void mm_kernel(uint8_t* lds, const uint8_t* __restrict__ raw, int N, int K,
                                 const signed char* __restrict__ aq, const float* __restrict__ asc,
                                 const short* __restrict__ absum, int M, int T, float* C, int ldc, int c_off, int accumulate,
                                 int s_begin, int s_end, const uint32_t* __restrict__ tabs) {
  constexpr int SB = MmT<QT>::SB;
  const int all = s_end - s_begin, slices = (all + SB - 1) / SB;
  const int groups = (N + 15) >> 4, gd = (int)gridDim.x;
  const int ng = (int)((long)(blockIdx.x + 1) * groups / gd) - (int)((long)blockIdx.x * groups / gd);
  float* GA = slices > 1 && ng <= MmL<QT>::GA ? (float*)(lds + SB * MmL<QT>::TOK + MM_WAVES * MmL<QT>::WSZ) : nullptr;
  if constexpr (QT == QT_IQ3_XXS) {  // (its codebook: the 256 words behind IQ3_S's)
    for (int i = threadIdx.x; i < 256; i += 512) ((uint32_t*)(lds + MmL<QT>::OGRID))[i] = tabs[512 + i];
  }
  if constexpr (QT == QT_IQ3_S) {  // (the codebook: the first 512 words of the tables; the first slice's meeting orders it)
    for (int i = threadIdx.x; i < 512; i += 512) ((uint32_t*)(lds + MmL<QT>::OGRID))[i] = tabs[i];
  }
  for (int sl = 0; sl < slices; ++sl) {
    if (sl) __syncthreads();  // (the tokens and partial sums of the slice before have been read)
    mm_slice<QT>(lds, raw, N, K, aq, asc, absum, M, T, C, ldc, c_off, GA ? accumulate : (accumulate || sl),
                 s_begin + all * sl / slices, s_begin + all * (sl + 1) / slices, GA, sl == 0, sl == slices - 1);
  }
}

#define MM_KERNEL(QTV)                                                                                                  \
  extern "C" __global__ __launch_bounds__(512, 1) void gemv_mm__QT##QTV(                                                \
      const uint8_t* __restrict__ raw, int N, int K, const uint32_t* tabs, const signed char* __restrict__ aq,          \
      const float* __restrict__ asc, const short* __restrict__ absum, int M, int T, float* C, int ldc, int c_off,       \
      int accumulate, int s_begin, int s_end) {                                                                         \
    __shared__ __attribute__((aligned(16))) uint8_t lds[MmL<QTV>::LDS];                                                 \
    /* gridDim.y > 1: K shared out over the work-groups (x, y), y-th of gridDim.y even pieces of the superblocks, the    \
       partial sums into plane y of C, here a workspace [gridDim.y][16][ldc] that gemv_mm_reduce adds up */              \
    const int ny = (int)gridDim.y, y = (int)blockIdx.y, all = s_end - s_begin;                                          \
    mm_kernel<QTV>(lds, raw, N, K, aq, asc, absum, M, T, C + (size_t)y * 16 * ldc, ldc, c_off, accumulate,              \
                   s_begin + all * y / ny, s_begin + all * (y + 1) / ny, tabs);                                         \
  }
MM_KERNEL(12)
MM_KERNEL(13)
MM_KERNEL(14)
MM_KERNEL(8)
MM_KERNEL(2)
MM_KERNEL(18)
MM_KERNEL(11)
MM_KERNEL(20)
MM_KERNEL(39)
MM_KERNEL(23)
MM_KERNEL(21)

// gemv_mm_reduce: C[t][c_off + n] (=, +=) the sum over the ny planes of ws [ny][16][N], plane 0 first, for the `rows`
// token rows a launch stores.  grid: ceil(rows * N / 256) work-groups of 256.
extern "C" __global__ __launch_bounds__(256) void gemv_mm_reduce(const float* __restrict__ ws, int ny, float* C, int rows, int N,
                                                                 int ldc, int c_off, int accumulate) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * N) return;
  const int t = i / N, n = i - t * N;
  float v = ws[(size_t)t * N + n];
  for (int y = 1; y < ny; ++y) v += ws[((size_t)y * 16 + t) * N + n];
  float* cp = C + (size_t)t * ldc + c_off + n;
  *cp = accumulate ? *cp + v : v;
}
