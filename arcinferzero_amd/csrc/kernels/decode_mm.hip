// "decode" module, part: gemv_mm, the matrix-vector form for 3..16 tokens on the matrix pipe (Q4_K).
//
// From a handful of tokens on, the dot-product GEMVs are bound by their vector ALU work (eight v_dot4 per token and
// 16-byte unit), not by memory, and past eight tokens the engine had only the prefill GEMM with its 64-token tiles.
// Here the int32 block sums come from v_mfma_i32_16x16x32_i8: a wave multiplies the 32 values of one block of 16
// weight rows with up to 16 tokens in one instruction, and the vector ALU is left with the f32 scale step of the
// prefill GEMM (reference zero/kernels/gemm.cl:454-469, 483):
//   res += (sa[t][b] * (d[n] * sc[n][b])) * (float)I[t][n][b]  -  (sa[t][b] * (float)S[t][b]) * (dmin[n] * mn[n][b])
// with S the sum of the block's 32 int8 activations.  The weights are read once, as in the GEMVs.
//
// Tokens.  A work-group of 8 waves stages superblocks [s_begin, s_end) of the tokens in LDS -- int8 rows, and per block
// the 16 tokens' sa and sa * S -- and keeps them for all its weight rows.  K in slices (s_begin, s_end) that fit LDS;
// later slices accumulate into C.
//
// Products.  Lane (n, g) = (lane % 16, lane / 16) is weight row n of a group of 16 rows as the instruction's column
// and supplies the 8 values 8 g .. 8 g + 7 of a block: bytes 8 g .. 8 g + 7 of a 32-byte chunk of Q4_K nibbles hold
// exactly those of the chunk's two blocks (low and high nibbles).  The instruction leaves the lane the sums of tokens
// 4 g .. 4 g + 3 with its row, whose scales it has decoded itself.  The min term of four blocks is one f32 matrix
// instruction (16 x 16 x 4) straight into the sums.
//
// Weights.  Were a lane to load the 8 bytes of a chunk that the matrix instruction wants from it, an instruction would
// touch 16 rows' lines for 32 bytes each: that form ran at 2 TB/s with or without its arithmetic.  Instead a lane
// loads 16 bytes such that eight lanes cover one row's superblock (a wave's instruction: 8 rows x 128 bytes), eight
// superblocks ahead in registers, and the wave turns a superblock's 2 KiB round through a piece of LDS of its own into
// the matrix instruction's layout (LDS operations of one wave complete in order: no barrier).  Headers come four
// superblocks at a time (lane (n, j): row n, superblock j of the four) through LDS in the same way.
//
// Work.  A work-group takes a contiguous run of 16-row groups (groups / gridDim.x of them, or one more); the run's
// (group, superblock) units, group-major, are cut into eight equal stretches, one per wave, so every wave streams the
// same amount whatever the number of groups.  A group that lies within one stretch is stored by its wave; one that is
// cut by a stretch boundary is added up after the work-group's one meeting, in wave order, by the wave in which it ends
// (it is that wave's first group).
#include "common.h"

#define MM_WAVES 8
#define MM_SPW 3  // slices of up to MM_WAVES * MM_SPW = 24 superblocks

typedef uint32_t mm_u2 __attribute__((ext_vector_type(2)));
typedef uint32_t mm_u4 __attribute__((ext_vector_type(4)));
struct MmSb { mm_u2 c[4]; mm_u4 h; };  // a lane's 8 bytes of each of a superblock's four chunks, the superblock's header

#define MM2_D 8  // superblocks in flight per wave

struct MmQ { mm_u4 a, b; };  // the lane's 16 bytes of a superblock of rows 0-7 and of rows 8-15 of the group

// one slice of K, superblocks [s_begin, s_end): at most MM_WAVES * MM_SPW of them
__device__ inline void mm_slice(uint8_t* lds, const uint8_t* __restrict__ raw, int N, int K,
                                const signed char* __restrict__ aq, const float* __restrict__ asc,
                                const short* __restrict__ absum, int M, int T, float* C, int ldc, int c_off, int accumulate,
                                int s_begin, int s_end, float* GA, bool first, bool last) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n16 = lane & 15, g = lane >> 4;
  const int nsb = K >> 8, sbs = s_end - s_begin, Ks = sbs * 256, nb = sbs * 8;
  uint8_t* A = lds;                            // [16][Ks] int8; 16-byte piece k of token t sits at piece k ^ t of its row
  float* SA = (float*)(lds + 16 * Ks);         // [nb][16] sa
  float* U = SA + nb * 16;                     // [nb][16] sa * S
  uint8_t* WB = (uint8_t*)(U + nb * 16);       // per wave: 2 KiB of nibbles, 1 KiB of headers
  uint8_t* WQ = WB + wave * 3072;
  uint8_t* WH = WQ + 2048;
  const PlanesQ4K pl = planes_q4k((size_t)N, nsb);
  const uint8_t* qs = raw + pl.qs;
  const uint8_t* hd = raw + pl.hdr;
  const int groups = (N + 15) >> 4, gd = (int)gridDim.x;
  const int gb0 = (int)((long)blockIdx.x * groups / gd), gb1 = (int)((long)(blockIdx.x + 1) * groups / gd);
  const int units = (gb1 - gb0) * sbs;         // >= 1: the grid has at most `groups` work-groups
  const int u0 = wave * units / MM_WAVES, u1 = (wave + 1) * units / MM_WAVES;
  const int ulast = max(u1 - 1, 0);            // (a wave without units loads unit 0 and drops it)
  // unit -> group of the run (units below 2^27): the high word of u * ceil(2^32 / sbs)
  const uint32_t magic = 0xFFFFFFFFu / (uint32_t)sbs + 1u;
  auto group_of = [&](int u) { return sbs == 1 ? u : (int)__umulhi((uint32_t)u, magic); };

  auto qload = [&](MmQ& q, int u) {  // u: the same in the whole wave, within the run
    const int gl = group_of(u), sb = u - gl * sbs;
    const int r0 = (gb0 + gl) * 16 + (lane >> 3);
    const size_t o = (size_t)(s_begin + sb) * 128 + (lane & 7) * 16;
    q.a = *(const mm_u4*)(qs + (size_t)min(r0, N - 1) * nsb * 128 + o);
    q.b = *(const mm_u4*)(qs + (size_t)min(r0 + 8, N - 1) * nsb * 128 + o);
  };
  auto hload = [&](mm_u4& h, int ub) {  // the headers of units ub .. ub + 3 (past the stretch: its last)
    const int u = min(ub + g, ulast);
    const int gl = group_of(u), sb = u - gl * sbs;
    const int r = min((gb0 + gl) * 16 + n16, N - 1);
    h = *(const mm_u4*)(hd + ((size_t)r * nsb + s_begin + sb) * 16);
  };

  // ---- staging.  Loads first: the tokens' int8 rows (wave w: rows 2 w and 2 w + 1, 16-byte pieces lane, lane + 64, ..),
  // their scales and sums (asc [K / 32][M], absum [K / 16][M]), then the wave's first superblocks right behind them:
  // loads come back in order, so the stores below wait for the tokens alone while the weights are on their way.
  constexpr int NCH = MM_WAVES * MM_SPW * 16 / 64;   // pieces per lane and row at most
  constexpr int NSC = MM_WAVES * MM_SPW * 8 * 16 / 512;  // (block, token) pairs per thread at most
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
    vu[i] = (int)absum[(size_t)(2 * b) * M + tt] + (int)absum[(size_t)(2 * b + 1) * M + tt];
  }
  __builtin_amdgcn_sched_barrier(0);
  MmQ q0, q1, q2, q3, q4, q5, q6, q7;
  mm_u4 hq0, hq1;
  hload(hq0, u0);
  hload(hq1, u0 + 4);
  qload(q0, min(u0 + 0, ulast));
  qload(q1, min(u0 + 1, ulast));
  qload(q2, min(u0 + 2, ulast));
  qload(q3, min(u0 + 3, ulast));
  qload(q4, min(u0 + 4, ulast));
  qload(q5, min(u0 + 5, ulast));
  qload(q6, min(u0 + 6, ulast));
  qload(q7, min(u0 + 7, ulast));
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
    U[idx] = sa * (float)vu[i];
  }
  __syncthreads();

  // the lane's places in the wave's LDS: piece p of row r of a superblock at 16-byte slot 16 p + (r ^ 2 p), so that the
  // writes (a quarter wave: two rows' eight pieces) and the reads (half a wave: one piece of 16 rows, 8 bytes a lane)
  // each go to all banks once
  const int wp = lane & 7, wr = lane >> 3;
  const int wa = (16 * wp + (wr ^ (2 * wp))) << 4, wb = wa ^ 128;
  int rd[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int p = 2 * c + (g >> 1);
    rd[c] = ((16 * p + (n16 ^ (2 * p))) << 4) + (g & 1) * 8;
  }
  const uint8_t* arow = A + n16 * Ks + (g & 1) * 8;

  // the products of one superblock (sbk: its index within the slice) of the lane's row, into acc
  auto products = [&](const MmSb& h, int sbk, v4f& acc) {
    const float d = f16_bits_to_f32(h.h.x), dmin = f16_bits_to_f32(h.h.x >> 16);
    const int b0 = sbk * 8;
    long av[8];
    float4 sa4[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      av[b] = *(const long*)(arow + ((sbk * 16 + ((2 * b + (g >> 1)) ^ n16)) << 4));
      sa4[b] = *(const float4*)(SA + (b0 + b) * 16 + 4 * g);
    }
    const float ua = U[(b0 + g) * 16 + n16], ub = U[(b0 + 4 + g) * 16 + n16];
    int sc[8], mn[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) q4k_scales_pair(h.h.y, h.h.z, h.h.w, j, sc[2 * j], sc[2 * j + 1], mn[2 * j], mn[2 * j + 1]);
    v4i I[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const mm_u2 cw = h.c[b >> 1];
      const uint32_t w0 = ((b & 1) ? cw.x >> 4 : cw.x) & 0x0F0F0F0Fu, w1 = ((b & 1) ? cw.y >> 4 : cw.y) & 0x0F0F0F0Fu;
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
  auto sbstep = [&](MmQ& q, int u, int j) {
    if (u < u1) {
      *(mm_u4*)(WQ + wa) = q.a;
      *(mm_u4*)(WQ + wb) = q.b;
    }
    qload(q, min(u + MM2_D, ulast));
    if (u < u1) {
      MmSb s;
#pragma unroll
      for (int c = 0; c < 4; ++c) s.c[c] = *(const mm_u2*)(WQ + rd[c]);
      s.h = *(const mm_u4*)(WH + ((j * 16 + n16) << 4));
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
#pragma unroll 1
  for (int u = u0; u < u1; u += 8) {
    *(mm_u4*)(WH + ((g * 16 + n16) << 4)) = hq0;
    hload(hq0, u + 8);
    sbstep(q0, u + 0, 0);
    sbstep(q1, u + 1, 1);
    sbstep(q2, u + 2, 2);
    sbstep(q3, u + 3, 3);
    *(mm_u4*)(WH + ((g * 16 + n16) << 4)) = hq1;
    hload(hq1, u + 12);
    sbstep(q4, u + 4, 0);
    sbstep(q5, u + 5, 1);
    sbstep(q6, u + 6, 2);
    sbstep(q7, u + 7, 3);
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
        const float* pw = (const float*)(WB + w * 3072) + (group_of(a0) == gf ? 0 : 256);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += pw[(4 * g + i) * 16 + n16];
      }
    }
    store(v, gf);
  }
}

// Superblocks [s_begin, s_end) of K, in slices of at most 24 that the work-group takes one after the other.  With more
// than one slice the sums of a work-group's groups wait in LDS for the last slice (up to MM_GA groups a work-group);
// with more groups than that a later slice adds to what the work-group itself has stored in C (other waves of it, as
// the stretches fall: the meetings between the slices order those stores and loads within the work-group).
#define MM_GA 12

extern "C" __global__ __launch_bounds__(512, 1) void gemv_mm__QT12(
    const uint8_t* __restrict__ raw, int N, int K, const uint32_t* tabs, const signed char* __restrict__ aq,
    const float* __restrict__ asc, const short* __restrict__ absum, int M, int T, float* C, int ldc, int c_off,
    int accumulate, int s_begin, int s_end) {
  // tokens 24 x (4096 + 1024) bytes at most, 3 KiB per wave, 1 KiB per group of sums
  __shared__ __attribute__((aligned(16))) uint8_t lds[MM_WAVES * MM_SPW * 5120 + MM_WAVES * 3072 + MM_GA * 1024];
  const int all = s_end - s_begin, slices = (all + MM_WAVES * MM_SPW - 1) / (MM_WAVES * MM_SPW);
  const int groups = (N + 15) >> 4, gd = (int)gridDim.x;
  const int ng = (int)((long)(blockIdx.x + 1) * groups / gd) - (int)((long)blockIdx.x * groups / gd);
  float* GA = slices > 1 && ng <= MM_GA ? (float*)(lds + MM_WAVES * MM_SPW * 5120 + MM_WAVES * 3072) : nullptr;
  for (int sl = 0; sl < slices; ++sl) {
    if (sl) __syncthreads();  // (the tokens and partial sums of the slice before have been read)
    mm_slice(lds, raw, N, K, aq, asc, absum, M, T, C, ldc, c_off, GA ? accumulate : (accumulate || sl),
             s_begin + all * sl / slices, s_begin + all * (sl + 1) / slices, GA, sl == 0, sl == slices - 1);
  }
}
