// "moe" module: routing, grouping of the (token, expert) pairs by expert, the expert-input quantizer and the final
// combine of a mixture-of-experts FFN (reference zero/kernels/moe.cl:50-179, 258-290, 344-352).  The reference
// compiles these with -DNE (experts), -DNU (experts per token), -DTM (slots per tile); here they are trailing
// arguments.
#include "quant.h"
#include "route1.h"


// moe_route: one wave per token.  The NU largest of NE logits (ties: the lower expert), p = exp(l - max),
// weights p / sum of the selected p; counts[t / NPART][e]++ per selection (NPART: the tokens of a chunk of the pair
// list, see moe_scan); sgate[t] = sigmoid(logit NE) when the row holds one.
// grid: ceil(T / 4) work-groups of 256 threads.
__device__ inline void moe_route_body(const float* __restrict__ logits, int ldl, int T, int* __restrict__ ids,
                                      float* __restrict__ wts, float* __restrict__ sgate, int* __restrict__ counts,
                                      int NE, int NU, int NPART, const RouteVariant rv) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  const float* lg = logits + (size_t)t * ldl;
  int mysel;
  float mywt;
  route_one_token(lg, NE, NU, lane, mysel, mywt, rv);
  if (lane < NU) {
    ids[(size_t)t * NU + lane] = mysel;
    wts[(size_t)t * NU + lane] = mywt;
    // (the counters of the token's chunk: many adds to one word from all over the chip queue up at the memory side)
    atomicAdd(&counts[(size_t)(t / NPART) * NE + mysel], 1);
  }
  if (lane == 0 && sgate) sgate[t] = route_sgate(lg, NE, ldl > NE, rv);
}
extern "C" __global__ __launch_bounds__(256) void moe_route(const float* __restrict__ logits, int ldl, int T,
                                                            int* __restrict__ ids, float* __restrict__ wts,
                                                            float* __restrict__ sgate, int* __restrict__ counts,
                                                            int NE, int NU, int NPART) {
  moe_route_body(logits, ldl, T, ids, wts, sgate, counts, NE, NU, NPART, RouteVariant());
}
// -DUSUM=1: the launch also writes au[b][m] = sa * S (ops.hip's act_usum: the same expression, the same bits) for the nblk
// 32-blocks of the chunk's M quantized rows -- asc [nblk][M], absum [2 nblk][M] -- which the expert tile kernels' ready-made
// forms take by DMA; no launch of its own for 12 bytes in and 4 out per token and block.
extern "C" __global__ __launch_bounds__(256) void moe_route__USUM1(const float* __restrict__ logits, int ldl, int T,
                                                                   int* __restrict__ ids, float* __restrict__ wts,
                                                                   float* __restrict__ sgate, int* __restrict__ counts,
                                                                   const float* __restrict__ asc,
                                                                   const short* __restrict__ absum, int M,
                                                                   float* __restrict__ au, int nblk, int NE, int NU,
                                                                   int NPART) {
  {  // (the nblk x M entries dealt to the work-groups in runs of consecutive tokens of a block: whole lines read and written;
     //  by the work-group's own four tokens the launch took 23 us instead of 11)
    const size_t total = (size_t)nblk * M;
    const size_t per = ((total + gridDim.x - 1) / gridDim.x + 255) / 256 * 256;
    const size_t e1 = min(total, (size_t)(blockIdx.x + 1) * per);
    for (size_t e = (size_t)blockIdx.x * per + threadIdx.x; e < e1; e += 256) {
      const size_t b = e / M, m = e - b * M;
      const float sa = asc[e];
      au[e] = sa * (float)((int)absum[(2 * b) * M + m] + (int)absum[(2 * b + 1) * M + m]);
    }
  }
  moe_route_body(logits, ldl, T, ids, wts, sgate, counts, NE, NU, NPART, RouteVariant());
}
// (-DESCALE: argument 7 is escale [NE]; -DROUTE_DS -DRSCALE=s: argument 7 is ebias [NE]; zero/engine_moe.h:113-116)
extern "C" __global__ __launch_bounds__(256) void moe_route__ESCALE1(const float* __restrict__ logits, int ldl, int T,
                                                                     int* __restrict__ ids, float* __restrict__ wts,
                                                                     float* __restrict__ sgate, int* __restrict__ counts,
                                                                     const float* __restrict__ escale, int NE, int NU,
                                                                     int NPART) {
  RouteVariant rv;
  rv.escale = escale;
  moe_route_body(logits, ldl, T, ids, wts, sgate, counts, NE, NU, NPART, rv);
}
extern "C" __global__ __launch_bounds__(256) void moe_route__ROUTE_DS1(const float* __restrict__ logits, int ldl, int T,
                                                                       int* __restrict__ ids, float* __restrict__ wts,
                                                                       float* __restrict__ sgate, int* __restrict__ counts,
                                                                       const float* __restrict__ ebias, int NE, int NU,
                                                                       int NPART, float rscale) {
  RouteVariant rv;
  rv.ebias = ebias;
  rv.rscale = rscale;
  moe_route_body(logits, ldl, T, ids, wts, sgate, counts, NE, NU, NPART, rv);
}

// moe_route1: a single token straight into NU one-slot tiles (no counts, scan or scatter).  One wave.
__device__ inline void moe_route1_body(const float* __restrict__ logits, float* __restrict__ sgate, int* __restrict__ tiles,
                                       int* __restrict__ stok, float* __restrict__ swt, int* __restrict__ inv, int NE,
                                       int NU, int has_gate, const RouteVariant rv) {
  const int lane = threadIdx.x & 63;
  int mysel;
  float mywt;
  route_one_token(logits, NE, NU, lane, mysel, mywt, rv);
  if (lane < NU) {
    tiles[1 + 3 * lane] = mysel;
    tiles[2 + 3 * lane] = lane;
    tiles[3 + 3 * lane] = 1;
    stok[lane] = 0;
    swt[lane] = mywt;
    inv[lane] = lane;
  }
  if (lane == 0) {
    tiles[0] = NU;
    if (sgate) sgate[0] = route_sgate(logits, NE, has_gate != 0, rv);
  }
}
extern "C" __global__ __launch_bounds__(64) void moe_route1(const float* __restrict__ logits, float* __restrict__ sgate,
                                                            int* __restrict__ tiles, int* __restrict__ stok,
                                                            float* __restrict__ swt, int* __restrict__ inv, int NE,
                                                            int NU, int has_gate) {
  moe_route1_body(logits, sgate, tiles, stok, swt, inv, NE, NU, has_gate, RouteVariant());
}
extern "C" __global__ __launch_bounds__(64) void moe_route1__ESCALE1(const float* __restrict__ logits, float* __restrict__ sgate,
                                                                     int* __restrict__ tiles, int* __restrict__ stok,
                                                                     float* __restrict__ swt, int* __restrict__ inv,
                                                                     const float* __restrict__ escale, int NE, int NU,
                                                                     int has_gate) {
  RouteVariant rv;
  rv.escale = escale;
  moe_route1_body(logits, sgate, tiles, stok, swt, inv, NE, NU, has_gate, rv);
}
extern "C" __global__ __launch_bounds__(64) void moe_route1__ROUTE_DS1(const float* __restrict__ logits, float* __restrict__ sgate,
                                                                       int* __restrict__ tiles, int* __restrict__ stok,
                                                                       float* __restrict__ swt, int* __restrict__ inv,
                                                                       const float* __restrict__ ebias, int NE, int NU,
                                                                       int has_gate, float rscale) {
  RouteVariant rv;
  rv.ebias = ebias;
  rv.rscale = rscale;
  moe_route1_body(logits, sgate, tiles, stok, swt, inv, NE, NU, has_gate, rv);
}

// moe_route_small: the routing of a pass of a few tokens in one work-group of 512 threads -- moe_route, moe_scan and
// moe_scatter in one launch, with the same results: wave w routes tokens w, w + 8, ... (as moe_route), then thread i places pair
// i = (token i / NU, expert sid[i]) in slot (pairs of lower experts) + (earlier pairs of the same expert), which is
// the scan's offset plus the scatter's rank in pair order, and the first pair of every expert writes the expert's
// tiles of up to TM slots after those of the lower experts.  n = T * NU <= 512.
extern "C" __global__ __launch_bounds__(512) void moe_route_small(const float* __restrict__ logits, int ldl, int T,
                                                                  int* __restrict__ ids, float* __restrict__ wts,
                                                                  float* __restrict__ sgate, int* __restrict__ tiles,
                                                                  int* __restrict__ stok, float* __restrict__ swt,
                                                                  int* __restrict__ inv, int NE, int NU, int TM) {
  __shared__ __attribute__((aligned(16))) int sid[512], ntile[512];
  __shared__ float sw[512];
  const int lane = threadIdx.x & 63, n = T * NU;
  for (int t = threadIdx.x >> 6; t < T; t += 8) {
    const float* lg = logits + (size_t)t * ldl;
    int mysel;
    float mywt;
    route_one_token(lg, NE, NU, lane, mysel, mywt);
    if (lane < NU) {
      sid[t * NU + lane] = mysel;
      sw[t * NU + lane] = mywt;
      ids[(size_t)t * NU + lane] = mysel;
      wts[(size_t)t * NU + lane] = mywt;
    }
    if (lane == 0 && sgate) sgate[t] = ldl > NE ? 1.0f / (1.0f + expf(-lg[NE])) : 0.0f;
  }
  if ((int)threadIdx.x >= n) sid[threadIdx.x] = 0x7FFFFFFF;  // (past the pairs: an expert no pair has, so that the
                                                             //  loops below can take the list four entries at a time)
  __syncthreads();
  const int i = threadIdx.x, n4 = (n + 3) & ~3;
  int e = -1, slot = 0, rank = 0, cnt = 0;
  if (i < n) {
    e = sid[i];
    for (int j = 0; j < n4; j += 4) {
      const int4 q = *(const int4*)&sid[j];
      const int ej[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        slot += ej[c] < e ? 1 : 0;
        cnt += ej[c] == e ? 1 : 0;
        rank += (ej[c] == e && j + c < i) ? 1 : 0;
      }
    }
    slot += rank;
    stok[slot] = i / NU;
    swt[slot] = sw[i];
    inv[i] = slot;
  }
  ntile[i] = (i < n && rank == 0) ? (cnt + TM - 1) / TM : 0;
  __syncthreads();
  if (i < n && rank == 0) {
    int tb = 0;
    for (int j = 0; j < n4; j += 4) {
      const int4 q = *(const int4*)&sid[j];
      const int4 nt4 = *(const int4*)&ntile[j];
      tb += (q.x < e ? nt4.x : 0) + (q.y < e ? nt4.y : 0) + (q.z < e ? nt4.z : 0) + (q.w < e ? nt4.w : 0);
    }
    for (int q = 0; q < ntile[i]; ++q) {
      int* tp = tiles + 1 + 3 * (tb + q);
      tp[0] = e;
      tp[1] = slot + q * TM;
      tp[2] = min(TM, cnt - q * TM);
    }
  }
  if (i == (n < 512 ? 511 : 0)) {  // (a thread without a pair, when there is one)
    int tot = 0;
    for (int j = 0; j < n4; j += 4) {
      const int4 nt4 = *(const int4*)&ntile[j];
      tot += nt4.x + nt4.y + nt4.z + nt4.w;
    }
    tiles[0] = tot;
  }
}

// The grouping of the (token, expert) pairs by expert is a counting sort over chunks of the pair list.  moe_route counts
// the pairs of each expert per chunk of TPC tokens (counts [chunks][NE]: the adds of a chunk go to words of its own, so
// the many adds of a long prompt do not queue up on NE words); moe_scan turns the counts into each chunk's first slot
// per expert; moe_scatter places a chunk's pairs.  Pair i of expert e lands at offs[e] + (pairs of e before i), so the
// layout is the pair order within each expert: the same on every run (the reference draws slots from an atomic
// counter, zero/kernels/moe.cl:171-179; its results do not depend on the order, its layout does).

// moe_scan: counts [NCH][NE] (NCH = the chunks of this call, from n pairs of NU per token and TPC tokens a chunk) ->
// offs[e] / cursor[e] (first slot of expert e), the tile list tiles[0] = number of tiles then (expert, first slot,
// rows <= TM) per tile, tstart[e] = first tile of expert e, tstart[NE] = the tile count; and in place of each count the
// chunk's first slot for that expert, counts[c][e] = offs[e] + pairs of e in chunks before c.
// One work-group of 1024 threads, NE <= 512: thread (p, e) = (tid / NE, tid % NE) sums the chunks c = p, p + P, ...
// (P = 1024 / NE), the experts' totals are scanned by waves (shuffles, one meeting), then every thread walks its chunks
// again.  The two walks are dependent chains of at most ceil(NCH / P) loads.
extern "C" __global__ __launch_bounds__(1024) void moe_scan(int* __restrict__ counts, int* __restrict__ offs,
                                                            int* __restrict__ cursor, int* __restrict__ tiles,
                                                            int* __restrict__ tstart, int NE, int TM, int NCH) {
  __shared__ int part[1024];      // [p][e]: pairs of expert e in the chunks of part p
  __shared__ int wsum[2][16];     // per wave: experts' pair and tile totals
  __shared__ int eoff[512];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int P = 1024 / NE, p = tid / NE, e = tid - p * NE;
  const bool live = p < P;
  // chunks are dealt to the parts in runs: part p takes chunks [p * cpp, min(NCH, (p + 1) * cpp))
  const int cpp = (NCH + P - 1) / P, c0 = p * cpp, c1 = min(NCH, c0 + cpp);
  // (the first eight chunks' counts are read together, one memory latency, and kept for the second walk)
  int v8[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) v8[k] = live && c0 + k < c1 ? counts[(size_t)(c0 + k) * NE + e] : 0;
  int tot = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) tot += v8[k];
  if (live)
    for (int c = c0 + 8; c < c1; ++c) tot += counts[(size_t)c * NE + e];
  part[tid] = live ? tot : 0;
  __syncthreads();
  // experts' totals and tile counts, scanned: thread e < NE
  int c = 0, nt = 0;
  if (tid < NE) {
    for (int q = 0; q < P; ++q) c += part[q * NE + tid];
    nt = (c + TM - 1) / TM;
  }
  int ic = c, it = nt;  // inclusive scans within the wave
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int oc = __shfl_up(ic, d, 64), ot = __shfl_up(it, d, 64);
    if (lane >= d) { ic += oc; it += ot; }
  }
  if (lane == 63) { wsum[0][wave] = ic; wsum[1][wave] = it; }
  __syncthreads();
  if (tid < NE) {
    int bc = 0, bt = 0;
    for (int w = 0; w < wave; ++w) { bc += wsum[0][w]; bt += wsum[1][w]; }
    const int off = bc + ic - c, toff = bt + it - nt;
    offs[tid] = off;
    cursor[tid] = off;
    tstart[tid] = toff;
    eoff[tid] = off;
    if (tid == NE - 1) tiles[0] = tstart[NE] = toff + nt;
    for (int i = 0; i < nt; ++i) {
      int* tp = tiles + 1 + 3 * (toff + i);
      tp[0] = tid;
      tp[1] = off + i * TM;
      tp[2] = min(TM, c - i * TM);
    }
  }
  __syncthreads();
  if (live) {
    int base = eoff[e];
    for (int q = 0; q < p; ++q) base += part[q * NE + e];
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (c0 + k < c1) {
        counts[(size_t)(c0 + k) * NE + e] = base;
        base += v8[k];
      }
    for (int cc = c0 + 8; cc < c1; ++cc) {
      const int v = counts[(size_t)cc * NE + e];
      counts[(size_t)cc * NE + e] = base;
      base += v;
    }
  }
}

// moe_scatter: work-group c places the pairs of chunk c (at most 512: TPC tokens of NU pairs).  Thread i takes pair
// i0 + i = (token, expert e): its slot is the chunk's first slot for e (cursor [chunks][NE], as moe_scan left it) plus
// the number of earlier pairs of e in the chunk, counted from the chunk's expert list in LDS four entries a read.  The
// chunk's row of `cursor` is cleared for the next layer's counts.  grid: chunks x 512 threads.
extern "C" __global__ __launch_bounds__(512) void moe_scatter(const int* __restrict__ ids, const float* __restrict__ wts,
                                                              int n, int* __restrict__ cursor, int* __restrict__ stok,
                                                              float* __restrict__ swt, int* __restrict__ inv, int NU,
                                                              int NE, int TPC) {
  __shared__ __attribute__((aligned(16))) int sid[512];
  const int i = threadIdx.x, i0 = blockIdx.x * TPC * NU, m = min(n - i0, TPC * NU);
  int e = 0x7FFFFFFF;  // (past the chunk's pairs: an expert no pair has)
  if (i < m) e = ids[i0 + i];
  sid[i] = e;
  int base = 0;
  if (i < m) base = cursor[(size_t)blockIdx.x * NE + e];
  __syncthreads();
  if (i < m) {
    int rank = 0;
    const int full = i & ~3;
    for (int j = 0; j < full; j += 4) {
      const int4 q = *(const int4*)&sid[j];
      rank += (q.x == e) + (q.y == e) + (q.z == e) + (q.w == e);
    }
    for (int j = full; j < i; ++j) rank += sid[j] == e;
    const int s = base + rank;
    stok[s] = (i0 + i) / NU;
    swt[s] = wts[i0 + i];
    inv[i0 + i] = s;
  }
  __syncthreads();  // (every base has been read)
  for (int k = i; k < NE; k += 512) cursor[(size_t)blockIdx.x * NE + k] = 0;
}

// moe_quant: h [S][F] f32 (S slot rows, the first n in use) -> hq [S][F] int8, hsc [F/32][S] f32 with row stride S;
// no sums (reference zero/kernels/moe.cl:258-274; FV: columns >= FV quantize as zeros).  The grid covers the rows in
// use in tiles of 64; rows of a tile at or past S are skipped.  grid (F/256, ceil(n/64)), local 256.
// moe_quant_sums: the same, and the sums of each 16 quantized values, hbs [F/16][S] int16 (the layout of the dense
// quantizer's sums), which the Q4_K tile GEMM of the down projection takes for its min term.
template <bool SUMS>
__device__ inline void moe_quant_body(const float* __restrict__ h, int F, int S, signed char* __restrict__ hq,
                                      float* __restrict__ hsc, short* __restrict__ hbs, int FV) {
  __shared__ float lasc[8][64];
  __shared__ short lsum[16][64];
  const int s = blockIdx.x, m0 = blockIdx.y * 64;
  const int lane16 = threadIdx.x & 15, rg = threadIdx.x >> 4;
#pragma unroll 1
  for (int p = 0; p < 4; ++p) {
    const int r = p * 16 + rg, m = m0 + r;
    float v[16];
    const int base = s * 256 + 16 * lane16;
    if (m < S) {
      const float4* src = (const float4*)(h + (size_t)m * F + base);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 f = src[i];
        v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
      }
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (base + i >= FV) v[i] = 0.0f;
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = 0.0f;
    }
    const float amax = block_amax(v, 1);
    uint4 pk;
    int sum;
    quant16(v, amax, pk, sum);
    if (m < S) *(uint4*)(hq + (size_t)m * F + base) = pk;
    if ((lane16 & 1) == 0) lasc[lane16 >> 1][r] = amax / 127.0f;
    if (SUMS) lsum[lane16][r] = (short)sum;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = threadIdx.x + 256 * i, b = idx >> 6, r = idx & 63;
    if (m0 + r < S) hsc[((size_t)s * 8 + b) * S + m0 + r] = lasc[b][r];
  }
  if (SUMS) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = threadIdx.x + 256 * i, b = idx >> 6, r = idx & 63;
      if (m0 + r < S) hbs[((size_t)s * 16 + b) * S + m0 + r] = lsum[b][r];
    }
  }
}
extern "C" __global__ __launch_bounds__(256) void moe_quant(const float* __restrict__ h, int F, int S,
                                                            signed char* __restrict__ hq, float* __restrict__ hsc,
                                                            int FV) {
  moe_quant_body<false>(h, F, S, hq, hsc, nullptr, FV);
}
extern "C" __global__ __launch_bounds__(256) void moe_quant_sums(const float* __restrict__ h, int F, int S,
                                                                 signed char* __restrict__ hq, float* __restrict__ hsc,
                                                                 short* __restrict__ hbs, int FV) {
  moe_quant_body<true>(h, F, S, hq, hsc, hbs, FV);
}

// moe_combine: x[t][c] += sum over k (in order) of y[inv[t * NU + k]][c]  (+ sgate[t] * sh[t][c] when there is a
// shared expert: sh non-null).  A thread takes four neighbouring columns (128-bit loads of the eight rows), N a
// multiple of 4.  grid (ceil(N / 1024) * 256, T), local (256, 1).
extern "C" __global__ __launch_bounds__(256) void moe_combine(float* __restrict__ x, const float* __restrict__ sh,
                                                              const float* __restrict__ sgate, const float* __restrict__ y,
                                                              const int* __restrict__ inv, int N, int NU) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * 4, t = blockIdx.y;
  if (c >= N) return;
  float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  for (int k = 0; k < NU; ++k) {
    const float4 a = *(const float4*)(y + (size_t)inv[t * NU + k] * N + c);
    v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
  }
  if (sh) {
    const float gt = sgate[t];
    const float4 a = *(const float4*)(sh + (size_t)t * N + c);
    v.x += gt * a.x; v.y += gt * a.y; v.z += gt * a.z; v.w += gt * a.w;
  }
  float4* xp = (float4*)(x + (size_t)t * N + c);
  float4 o = *xp;
  o.x += v.x; o.y += v.y; o.z += v.z; o.w += v.w;
  *xp = o;
}
