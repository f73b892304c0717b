// "moe" module: routing, grouping of the (token, expert) pairs by expert, the expert-input quantizer and the final
// combine of a mixture-of-experts FFN (reference zero/kernels/moe.cl:50-179, 258-290, 344-352).  The reference
// compiles these with -DNE (experts), -DNU (experts per token), -DTM (slots per tile); here they are trailing
// arguments.
#include "quant.h"
#include "route1.h"


// moe_route: one wave per token.  The NU largest of NE logits (ties: the lower expert), p = exp(l - max),
// weights p / sum of the selected p; counts[copy][e]++ per selection (NPART copies [NPART][NE], 1 by default); sgate[t] = sigmoid(logit NE) when the row holds one.
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
    // (NPART copies of the counters, a work-group adding to copy blockIdx % NPART: many adds to one word from all
    //  over the chip queue up at the memory side; moe_scan sums the copies)
    atomicAdd(&counts[(size_t)(blockIdx.x % NPART) * NE + mysel], 1);
  }
  if (lane == 0 && sgate) sgate[t] = route_sgate(lg, NE, ldl > NE, rv);
}
extern "C" __global__ __launch_bounds__(256) void moe_route(const float* __restrict__ logits, int ldl, int T,
                                                            int* __restrict__ ids, float* __restrict__ wts,
                                                            float* __restrict__ sgate, int* __restrict__ counts,
                                                            int NE, int NU, int NPART) {
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

// moe_scan: exclusive scan of the counts -> offs / cursor; the tile list tiles[0] = number of tiles, then (expert,
// first slot, rows <= TM) per tile; tstart[e] = first tile of expert e, tstart[NE] = the tile count; counts (all NPART copies) reset.
// One work-group of 1024 threads (NE <= 1024).
extern "C" __global__ __launch_bounds__(1024) void moe_scan(int* __restrict__ counts, int* __restrict__ offs,
                                                            int* __restrict__ cursor, int* __restrict__ tiles,
                                                            int* __restrict__ tstart, int NE, int TM, int NPART) {
  __shared__ int a[1024], b[1024];
  const int e = threadIdx.x;
  // the copies moe_route counted into, summed (integer adds in LDS: any order gives the same sums) and reset
  a[e] = 0;
  __syncthreads();
  for (int i = e; i < NPART * NE; i += 1024) {
    atomicAdd(&a[i % NE], counts[i]);
    counts[i] = 0;
  }
  __syncthreads();
  const int c = e < NE ? a[e] : 0, nt = (c + TM - 1) / TM;
  __syncthreads();
  a[e] = c;
  b[e] = nt;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int x = e >= d ? a[e - d] : 0, y = e >= d ? b[e - d] : 0;
    __syncthreads();
    a[e] += x;
    b[e] += y;
    __syncthreads();
  }
  if (e >= NE) return;
  const int off = a[e] - c, toff = b[e] - nt;
  offs[e] = off;
  cursor[e] = off;
  tstart[e] = toff;
  if (e == NE - 1) tiles[0] = tstart[NE] = b[e];
  for (int i = 0; i < nt; ++i) {
    int* tp = tiles + 1 + 3 * (toff + i);
    tp[0] = e;
    tp[1] = off + i * TM;
    tp[2] = min(TM, c - i * TM);
  }
}

// moe_scatter: places pair i = (token i / NU, expert ids[i]) in a slot of its expert's range, in pair order: the
// k-th pair of expert e (counting i upwards) gets slot offs[e] + k, so the layout is the same on every run (the
// reference draws slots from an atomic counter; its results do not depend on the order, its layout does).
// One work-group of 256 threads per expert, each scanning all n pairs.  `cursor` holds offs (as moe_scan wrote it).
// The list is taken in pieces of 256 * SCAT_IT pairs: first every wave counts its matches in each 256-pair step of the
// piece (no barrier between steps), then one scan over the (step, wave) counts gives every wave its first rank in
// every step, then the steps are run again and the pairs written.
#define SCAT_IT 32
extern "C" __global__ __launch_bounds__(256) void moe_scatter(const int* __restrict__ ids, const float* __restrict__ wts,
                                                              int n, int* __restrict__ cursor, int* __restrict__ stok,
                                                              float* __restrict__ swt, int* __restrict__ inv, int NU) {
  __shared__ int cnt[SCAT_IT * 4];  // matches of wave w in step j at [4 j + w], then their exclusive prefix sums
  __shared__ int wtot[4];
  const int e = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  int base = cursor[e];
  for (int p0 = 0; p0 < n; p0 += 256 * SCAT_IT) {
    int my[SCAT_IT];  // the thread's pairs of the piece, all loads in flight together
#pragma unroll
    for (int j = 0; j < SCAT_IT; ++j) {
      const int i = p0 + j * 256 + t;
      my[j] = i < n ? ids[i] : -1;
    }
#pragma unroll
    for (int j = 0; j < SCAT_IT; ++j) {
      const unsigned long long bal = __ballot(my[j] == e);
      if (lane == 0) cnt[4 * j + wave] = __popcll(bal);
    }
    __syncthreads();
    // exclusive scan of cnt[0 .. 4 SCAT_IT): threads 0-63 own entries 2 t, 2 t + 1, the rest none
    int c0 = 0, c1 = 0;
    if (t < 2 * SCAT_IT) { c0 = cnt[2 * t]; c1 = cnt[2 * t + 1]; }
    int incl = c0 + c1;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(incl, d, 64);
      if (lane >= d) incl += o;
    }
    if (lane == 63) wtot[wave] = incl;
    __syncthreads();
    int before = 0;
    for (int w = 0; w < wave; ++w) before += wtot[w];
    const int total = wtot[0] + wtot[1] + wtot[2] + wtot[3];
    const int excl = before + incl - (c0 + c1);
    if (t < 2 * SCAT_IT) { cnt[2 * t] = excl; cnt[2 * t + 1] = excl + c0; }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < SCAT_IT; ++j) {
      const int i = p0 + j * 256 + t;
      const bool mine = my[j] == e;
      const unsigned long long bal = __ballot(mine);
      if (mine) {
        const int s = base + cnt[4 * j + wave] + __popcll(bal & ((1ull << lane) - 1));
        stok[s] = i / NU;
        swt[s] = wts[i];
        inv[i] = s;
      }
    }
    base += total;
    __syncthreads();  // (cnt and wtot are rewritten by the next piece)
  }
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
