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
// Mapping.  A work-group of 8 waves stages superblocks [s_begin, s_end) of the tokens in LDS -- int8 rows with a
// 16-byte pad, and per block the 16 tokens' sa and sa * S -- then takes groups of 16 weight rows in turn.  Within a
// group the waves share out K in superblocks (wave w: w, w + 8, ...: a wave's four 8-byte loads of a row's superblock
// fall into one 128-byte line, back to back) and meet once per group to add their partial sums in a fixed order.
// Lane (n, g) = (lane % 16, lane / 16) is weight row n of the group as the instruction's column and supplies the 8
// values 8 g .. 8 g + 7 of a block: bytes 8 g .. 8 g + 7 of a 32-byte chunk of Q4_K nibbles hold exactly those of the
// chunk's two blocks (low and high nibbles), so a lane loads 8 bytes per chunk and nothing moves between lanes.  The
// instruction leaves the lane the sums of tokens 4 g .. 4 g + 3 with its row, whose scales it has decoded itself.  The
// min term of four blocks is one f32 matrix instruction (16 x 16 x 4) straight into the sums.  The next group's loads
// are in flight while the current group is computed.  K in slices (s_begin, s_end) that fit LDS; later slices
// accumulate into C.
#include "common.h"

#define MM_WAVES 8
#define MM_SPW 3  // superblocks per wave and slice at most: slices of up to 24 superblocks

typedef uint32_t mm_u2 __attribute__((ext_vector_type(2)));
typedef uint32_t mm_u4 __attribute__((ext_vector_type(4)));
struct MmSb { mm_u2 c[4]; mm_u4 h; };  // the four chunks' 8 bytes each, the superblock's header

__device__ inline void mm_load(MmSb (&r)[MM_SPW], const uint8_t* __restrict__ raw, const PlanesQ4K& pl, int nsb, int row,
                               int g, int wave, int s_begin, int sbs) {
#pragma unroll
  for (int k = 0; k < MM_SPW; ++k) {
    const int sb = s_begin + min(wave + MM_WAVES * k, sbs - 1);  // (past the slice: clamped, its terms dropped)
    const uint8_t* q = raw + pl.qs + ((size_t)row * nsb + sb) * 128 + 8 * g;
#pragma unroll
    for (int c = 0; c < 4; ++c) r[k].c[c] = *(const mm_u2*)(q + 32 * c);
    r[k].h = *(const mm_u4*)(raw + pl.hdr + ((size_t)row * nsb + sb) * 16);
  }
}

extern "C" __global__ __launch_bounds__(512, 1) void gemv_mm__QT12(
    const uint8_t* __restrict__ raw, int N, int K, const uint32_t* tabs, const signed char* __restrict__ aq,
    const float* __restrict__ asc, const short* __restrict__ absum, int M, int T, float* C, int ldc, int c_off,
    int accumulate, int s_begin, int s_end) {
  // (sized for the largest slice, MM_WAVES * MM_SPW superblocks: 16 (6144 + 16) + 2 * 192 * 16 * 4 + 2 * 8192 bytes)
  __shared__ __attribute__((aligned(16))) uint8_t lds[16 * (MM_WAVES * MM_SPW * 256 + 16) + 2 * MM_WAVES * MM_SPW * 8 * 16 * 4 + 2 * MM_WAVES * 256 * 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n16 = lane & 15, g = lane >> 4;
  const int nsb = K >> 8, sbs = s_end - s_begin, Ks = sbs * 256, nb = sbs * 8;
  const int astride = Ks + 16;
  uint8_t* A = lds;                                // [16][Ks + 16] int8
  float* SA = (float*)(lds + 16 * astride);        // [nb][16] sa
  float* U = SA + nb * 16;                         // [nb][16] sa * S
  float* RED = U + nb * 16;                        // two copies of [MM_WAVES][16 tokens][16 rows]
  const PlanesQ4K pl = planes_q4k((size_t)N, nsb);
  const int groups = (N + 15) >> 4;

  // (two buffers with fixed names -- one chosen by a run-time index would live in memory: the next group is in flight
  //  while a group is computed)
  MmSb ra[MM_SPW], rb[MM_SPW];
  int grp = blockIdx.x;
  const int gd = (int)gridDim.x;

  // ---- staging: wave w takes token rows 2 w and 2 w + 1 (tokens from T on: zeros), a lane their 16-byte chunks lane,
  // lane + 64, ...; all loads first (an index past the row's end is clamped: the lanes that get the same chunk store
  // the same bytes), so the staging costs one memory latency.  Per block the tokens' scale and scaled sum of the 32
  // values (the two lanes of a block add their halves' sums).
  {
    constexpr int NCH = MM_WAVES * MM_SPW * 16 / 64;  // chunks per lane and row at most
    const int cpr = Ks >> 4;                          // chunks per row (even)
    mm_u4 va[2][NCH];
    float vs[2][NCH];
#pragma unroll
    for (int r2 = 0; r2 < 2; ++r2) {
      const int t = 2 * wave + r2, tt = t < T ? t : 0;
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int k16 = min(lane + 64 * i, cpr - 1);
        va[r2][i] = *(const mm_u4*)(aq + (size_t)tt * K + (size_t)s_begin * 256 + k16 * 16);
        vs[r2][i] = asc[(size_t)(s_begin * 8 + (k16 >> 1)) * M + tt];
      }
    }
    // the first group's rows right behind the staging loads: loads come back in order, so the stores below wait for
    // the tokens alone while the rows are on their way (the other way round the tokens queued behind 12 MB of rows)
    __builtin_amdgcn_sched_barrier(0);
    mm_load(ra, raw, pl, nsb, min(min(grp, groups - 1) * 16 + n16, N - 1), g, wave, s_begin, sbs);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r2 = 0; r2 < 2; ++r2) {
      const int t = 2 * wave + r2;
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int k16 = min(lane + 64 * i, cpr - 1);
        mm_u4 v = va[r2][i];
        float sa = vs[r2][i];
        if (t >= T) { v = mm_u4{0, 0, 0, 0}; sa = 0.0f; }
        *(mm_u4*)(A + t * astride + k16 * 16) = v;
        int sm = dot4(v.x, 0x01010101u, 0);
        sm = dot4(v.y, 0x01010101u, sm);
        sm = dot4(v.z, 0x01010101u, sm);
        sm = dot4(v.w, 0x01010101u, sm);
        // (the block's other half is the neighbouring lane's chunk; for the clamped lanes of the last chunk, an odd
        //  one, the neighbour holds the same chunk and they are not the ones that store)
        sm += __shfl_xor(sm, 1, 64);
        if ((k16 & 1) == 0) {
          SA[(k16 >> 1) * 16 + t] = sa;
          U[(k16 >> 1) * 16 + t] = sa * (float)sm;
        }
      }
    }
  }
  __syncthreads();

  // one group: the next one's loads go out into `next`, then the products of `cur`
  int parity = 0;
  auto step = [&](const MmSb (&cur)[MM_SPW], MmSb (&next)[MM_SPW]) {
    // (unconditional: past the last group the last one is loaded again and never used, so the number of loads in
    //  flight is the same on every path)
    const int nxt = min(grp + gd, groups - 1);
    mm_load(next, raw, pl, nsb, min(nxt * 16 + n16, N - 1), g, wave, s_begin, sbs);
    __builtin_amdgcn_sched_barrier(0);
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int k = 0; k < MM_SPW; ++k) {
      const int sbk = wave + MM_WAVES * k;
      if (sbk < sbs) {  // (the same for the whole wave)
        const MmSb& h = cur[k];
        const float d = f16_bits_to_f32(h.h.x), dmin = f16_bits_to_f32(h.h.x >> 16);
        const int b0 = sbk * 8;  // first of the superblock's eight blocks, within the slice
        // the tokens' operands of all eight blocks first, then the eight matrix instructions back to back, then the
        // scale steps: block by block, every step would wait out the latency of its LDS read and of its instruction
        long av[8];
        float4 sa4[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) {
          av[b] = *(const long*)(A + n16 * astride + (b0 + b) * 32 + 8 * g);
          sa4[b] = *(const float4*)(SA + (b0 + b) * 16 + 4 * g);
        }
        const float u0 = U[(b0 + g) * 16 + n16], u1 = U[(b0 + 4 + g) * 16 + n16];
        int sc[8], mn[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) q4k_scales_pair(h.h.y, h.h.z, h.h.w, j, sc[2 * j], sc[2 * j + 1], mn[2 * j], mn[2 * j + 1]);
        __builtin_amdgcn_sched_barrier(0);
        v4i I[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) {  // chunk b / 2: its low nibbles are block b (even), its high ones block b (odd)
          const mm_u2 cw = h.c[b >> 1];
          const uint32_t w0 = ((b & 1) ? cw.x >> 4 : cw.x) & 0x0F0F0F0Fu, w1 = ((b & 1) ? cw.y >> 4 : cw.y) & 0x0F0F0F0Fu;
          const long wv = (long)(((unsigned long)w1 << 32) | w0);
          v4i z = {0, 0, 0, 0};
          I[b] = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[b], wv, z, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
          const float ws = d * (float)sc[b];
          acc[0] = fmaf((float)I[b][0], sa4[b].x * ws, acc[0]);
          acc[1] = fmaf((float)I[b][1], sa4[b].y * ws, acc[1]);
          acc[2] = fmaf((float)I[b][2], sa4[b].z * ws, acc[2]);
          acc[3] = fmaf((float)I[b][3], sa4[b].w * ws, acc[3]);
        }
        // the min term of each half's four blocks, - sum_b (sa S)[t][b] (dmin mn)[n][b], as one f32 matrix instruction
        // straight into the sums: lane (n, g) supplies its row's factor of block 4 hh + g and token n's of that block
        const int m0 = g == 0 ? mn[0] : g == 1 ? mn[1] : g == 2 ? mn[2] : mn[3];
        const int m1 = g == 0 ? mn[4] : g == 1 ? mn[5] : g == 2 ? mn[6] : mn[7];
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(u0, -(dmin * (float)m0), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(u1, -(dmin * (float)m1), acc, 0, 0, 0);
      }
    }
    // the waves' partial sums of the group, added in wave order (two copies of RED in turn: one meeting per group)
    float* red = RED + parity * (MM_WAVES * 256);
    parity ^= 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) red[(wave * 16 + 4 * g + i) * 16 + n16] = acc[i];
    __syncthreads();
    if (tid >= 256) {  // (the upper four waves: the ones with fewer superblocks when these do not divide by 8)
      const int t = (tid - 256) >> 4, n = grp * 16 + (tid & 15);
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < MM_WAVES; ++w) v += red[(w * 16 + t) * 16 + (tid & 15)];
      if (t < (T > 8 ? 16 : T) && n < N) {  // (9-16 tokens: the chunk has 16 rows, those from T on come out as zeros)
        float* cp = C + (size_t)t * ldc + c_off + n;
        if (accumulate) v += *cp;
        *cp = v;
      }
    }
  };
  while (grp < groups) {
    step(ra, rb);
    grp += gd;
    if (grp >= groups) break;
    step(rb, ra);
    grp += gd;
  }
}
