/*
 * CPU oracle for the GGUF block-quantized matmul path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference engine for the path this repository accelerates.
 * It is the checker that tests, the smoke check and the bench's cpu_baseline leg compare the HIP kernels with;
 * nothing in the shipped library links, loads or calls it.
 *
 * Every function names the reference lines it follows (paths relative to the reference tree).
 *
 * Pin status (what holds each function to the reference, see tests/test_oracle_*.py):
 *   orc_fp16_to_f32 / orc_f32_to_fp16   all 65,536 patterns vs numpy.float16; random + tie f32 inputs vs numpy and
 *                                       vs the compiled reference header (oracle/_ref)
 *   orc_decode_sb / orc_dequant_row     closed-form blocks with exact binary fractions; pack/unpack brute force;
 *                                       golden vectors and live comparison with the compiled reference header
 *   orc_quantize_act                    closed forms (max -> +-127, zero block, ties to even); golden + compiled ref
 *   orc_quantize_rows_q8_0              golden + compiled ref; round trip bound
 *   orc_act_residual                    PARITY UNPINNED (no reference CPU twin, no vector); identities and bounds only
 *   orc_quantize_rows_q4_0, Q4_0 decode  closed-form blocks; live comparison with the compiled reference header
 *   IQ4_XS decode                       closed-form block; live comparison with the compiled reference header
 *   IQ3_XXS decode (and its grid table) closed-form block; live comparison with the compiled reference header over every
 *                                       grid index and on blocks of random bytes
 *   Q3_K decode                         closed-form block; live comparison with the compiled reference header
 *   IQ4_NL, MXFP4 decode                closed-form blocks (every code, every E8M0 exponent); live comparison with the
 *                                       compiled reference header
 *   AR4_128, Q2_0 decode                closed-form blocks (every code at every position); golden vectors
 *                                       (tests/golden/ref_vectors_types4.npz) and live comparison with the compiled
 *                                       reference header
 *   IQ3_S decode (and its grid table)   closed-form block; golden vectors (tests/golden/ref_vectors_types2.npz) and live
 *                                       comparison with the compiled reference header over every grid index
 *   Q5_K decode                         closed-form block; golden vectors (tests/golden/ref_vectors_q5k.npz) and live
 *                                       comparison with the compiled reference header
 *   orc_block_sums                      brute-force integer sums in numpy (int64)
 *   orc_matmul_ref                      numpy float64 dot of dequantized rows; unit-scale known answer
 *   orc_matmul_formula                  against orc_matmul_ref within float rounding; unit-scale known answer (exact)
 *   orc_moe_route                       stable-sort top-k in numpy (the reference's own CPU check, tests/test_route.cpp:28-44)
 *   orc_moe_scan / orc_moe_scatter      invariants (bijection, contiguity, counts) + numpy restatement
 *   orc_moe_layer                       composition of the above, compared with a numpy float64 composition
 * The f32 -> Q4_K / Q5_K / Q6_K / IQ4_XS quantizers used to make synthetic weights are not part of the reference (it has none) and
 * not part of this file: they are input generators of the product's bench/test utilities; parity unpinned by design.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_Q4_0 2u
#define ORC_Q8_0 8u
/* Q4_0 is Q8_0 with q - 8 in four bits (src/quants.h:136): everything after the decode treats the two alike */
/* IQ4_NL and MXFP4 are Q4_0 with a table of 16 values in the place of q - 8 (and MXFP4 a power-of-two scale byte in the
 * place of the f16 one): src/quants.h:520-530, 594-606 */
#define ORC_IQ4_NL 20u
#define ORC_MXFP4 39u
/* AR4_128 is Q4_0 with one f16 scale for four 32-blocks; Q2_0 has 64-blocks of 2-bit codes q, value d * (q - 1):
 * src/quants.h:531-542, 607-616 */
#define ORC_AR4_128 0x41523447u
#define ORC_Q2_0 42u
#define ORC_Q8LIKE(t) \
  ((t) == ORC_Q8_0 || (t) == ORC_Q4_0 || (t) == ORC_IQ4_NL || (t) == ORC_MXFP4 || (t) == ORC_AR4_128 || (t) == ORC_Q2_0)
#define ORC_Q4_K 12u
#define ORC_Q5_K 13u
#define ORC_Q45(t) ((t) == ORC_Q4_K || (t) == ORC_Q5_K) /* d, dmin, 6-bit scales and mins */
#define ORC_Q6_K 14u
#define ORC_IQ4_XS 23u
/* one int scale per 16 (Q6_K) or per 32 values (IQ4_XS: the same one for both halves), kept in sc6[], and no mins */
#define ORC_IQ3_S 21u
#define ORC_Q3_K 11u /* 3-bit values - 4 with a 6-bit scale - 32 per 16 of them: q[] and sc6[] as the IQ types' */
#define ORC_IQ3_XXS 18u
#define ORC_IQLIKE(t) ((t) == ORC_IQ4_XS || (t) == ORC_IQ3_S || (t) == ORC_Q3_K || (t) == ORC_IQ3_XXS) /* q[] holds the signed value itself */
#define ORC_Q6LIKE(t) ((t) == ORC_Q6_K || ORC_IQLIKE(t))

/* ---------------------------------------------------------------- fp16 (src/quants.h:17-52) */

/* IEEE binary16 -> f32, exact; subnormals normalized (src/quants.h:17-31). */
float orc_fp16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu, bits;
  if (e == 0) {
    if (m == 0) {
      bits = sign;
    } else {
      int ex = 127 - 15 + 1;
      while (!(m & 0x400u)) { m <<= 1; --ex; }
      bits = sign | ((uint32_t)ex << 23) | ((m & 0x3FFu) << 13);
    }
  } else if (e == 31) {
    bits = sign | 0x7F800000u | (m << 13);
  } else {
    bits = sign | ((e + 127 - 15) << 23) | (m << 13);
  }
  float r;
  memcpy(&r, &bits, 4);
  return r;
}

/* f32 -> binary16, round to nearest even, NaN -> quiet, overflow -> inf, below 2^-25 -> signed zero
 * (src/quants.h:33-52). */
uint16_t orc_f32_to_fp16(float x) {
  uint32_t f;
  memcpy(&f, &x, 4);
  const uint32_t sign = (f >> 16) & 0x8000u;
  const uint32_t e8 = (f >> 23) & 0xFFu;
  uint32_t mant = f & 0x7FFFFFu;
  const int32_t e = (int32_t)e8 - 127 + 15;
  if (e8 == 0xFF) return (uint16_t)(sign | 0x7C00u | (mant ? 0x200u : 0u));
  if (e >= 31) return (uint16_t)(sign | 0x7C00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)sign;
    mant |= 0x800000u;
    const uint32_t shift = (uint32_t)(14 - e);
    uint32_t h = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1u))) ++h;
    return (uint16_t)(sign | h);
  }
  uint32_t h = sign | ((uint32_t)e << 10) | (mant >> 13);
  const uint32_t rem = mant & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
  return (uint16_t)h;
}

/* ---------------------------------------------------------------- block formats (src/gguf.h:48-79) */

/* Bytes of one 256-element superblock in GGUF (src/gguf.h:59,62,64; src/quants.h:327-331). 0 = unsupported. */
int orc_sb_bytes(uint32_t type) {
  switch (type) {
    case ORC_Q8_0: return 34 * 8;
    case ORC_Q4_0: return 18 * 8;
    case ORC_IQ4_NL: return 18 * 8;
    case ORC_MXFP4: return 17 * 8;
    case ORC_AR4_128: return 66 * 2;
    case ORC_Q2_0: return 18 * 4;
    case ORC_Q4_K: return 144;
    case ORC_Q5_K: return 176;
    case ORC_Q6_K: return 210;
    case ORC_IQ4_XS: return 136;
    case ORC_IQ3_S: return 110;
    case ORC_Q3_K: return 110;
    case ORC_IQ3_XXS: return 98;
    default: return 0;
  }
}

/* 6-bit scale / min of sub-block j of a Q4_K superblock from its 12 packed bytes (src/quants.h:61-69). */
static void scale_min_k4(int j, const uint8_t* q, int* sc, int* mn) {
  if (j < 4) {
    *sc = q[j] & 63;
    *mn = q[j + 4] & 63;
  } else {
    *sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
    *mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
  }
}

/*
 * One decoded superblock (the fields of the reference's DecodedSB that the three types use, src/quants.h:72-84).
 *   Q4_K: q 0..15, sc[8], mn[8], d, dmin        (src/quants.h:91-113)
 *   Q5_K: the same with q 0..31                  (src/quants.h:101-108)
 *   Q6_K: q 0..63 (offset 32 NOT removed), sc6[16], d   (src/quants.h:115-134)
 *   Q8_0: q -128..127, d8[8]                    (src/quants.h:149-157)
 *   IQ4_XS: q = the 16-entry table's value of each 4-bit code, sc6[2 b] = sc6[2 b + 1] = the block's 6-bit scale - 32,
 *           d                                   (src/quants.h:297-311; the table: src/iq_tables.h:364-367)
 */
static const int8_t iq4_values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* The IQ3_S codebook (ggml's iq3s_grid, a constant of the GGUF format; the reference carries it as
 * src/iq_tables.h:297): 512 groups of four magnitudes, each one of 1, 3, ..., 15.  Kept as three hex digits per entry,
 * magnitude j = 2 * ((code >> 3 j) & 7) + 1. */
static const char iq3s_codes[] =
"00000100200500700800900a00c00e01001101501b02002202502702902b03003203903c03f04004104204404804904d"
"05005305705905d06407107507a08008108508708808b08e09109509809c0a20a50a70a90ab0b80bb0c30c90cd0d00d2"
"0d90db0de0e40e80ea0f70f90fd10010b10f11111411a12012312913814214415015215615b16116516717617b186189"
"18b1991aa1b91c01c21c41d01d21d61db1e81ec20020120220420820920b20d20f21021221921c21e22c22e23123a240"
"24124324624824c25125825b26126826a27827e28028a28d28f29029429a2a02a32ad2b02ba2c12c42c72c82cb2d12d7"
"2d82dc2e12f22f830330530a30c31931b32232632832c34134834b35135835a3693903943973a43a63c13c33c83ca3d1"
"3dd3e13f23f840040140340540740840a40c40e41141341741841a42142342542842a43743843b43d44044244844b44f"
"45245545945c46246948148448749149349849f4a14ab4af4b94bc4c04c24c54c94d24d44d94db4e24e84f6501507510"
"51351a51d52153a53d54454955255f56056b5785805825875915ad5b15c55c95d65d85e35e860260960b60d60f612619"
"61b61d62262462762963363964164364564c65165366067067a67e68068a69069a69c6a86c16c86cc6d16d36d76d86e1"
"6e36e76ed6fb70370970e71271972a73073474174874a75575a76476e77b78e7a17c17c37d07d27dd80080480a810814"
"81781a82182883884284784984b85285885d86386986d88188388888d89189b8a08af8b28b88c48c98cb8d08d28d98dd"
"90090291491f92093994594795197298b99c9b09c89cd9d89e39e9a02a08a0ca12a20a24a27a2aa36a3ca41a43a45a4a"
"a51a5aa7aa80a89a93a98a9eaabac2ac7ac8ad7ae4ae9af5afbb01b04b10b1ab26b4ab56b69b6bba2bc2bc4bd2c09c0b"
"c0dc19c1bc30c40c50c57c74c8ac9cca2cadcb2cb8cc0ccccd1ce0d15d23d32d40d43d5cd70d85da0dc9dcbe00e04e07"
"e10e12e1ee20e2ce32e42e49e54e63e65e81e84e88e8ee91e98ea9ec2edaeddeebf01f05f0bf10f28f52f62f82f99fc0";
/* The IQ3_XXS codebook (ggml's iq3xxs_grid, a constant of the GGUF format; the reference carries it in
 * src/iq_tables.h): 256 entries of four magnitudes out of 4, 12, 20, 28, 36, 44, 52, 62, here three hex digits an
 * entry, magnitude j its bits 3 j .. 3 j + 2 as an index into that list. */
static const char iq3xxs_codes[] =
"00000200400900b00f01001201902203b03d04104304804a05105505805a06106c07808008208408909009209909b09f"
"0a90af0bd0c10c70c80ca0d50f810b11f12412f13b13d14114715a16a19d1b41c81cc1ce1e31f120120320820a211213"
"21821a21c22722824024224925025228128328828a2912982ba2c02c22d02d92e62f63013053283503543663793853d2"
"3e040040240940b41041241641942244144344544844a45145847347747848048248948f49049249f4a04ad4c14c84cc"
"4f84fc51d52b54355756157c5c15c35ce5e560160860a61161362863563a6406426506596646666816836886956aa6ba"
"6c96db71872773a74074675276d78c79e7b37db7f080480f81d81f82b82f87c89089f8a08b08b68c78e5904929934955"
"9639789c59c89ca9d8a0aa21a38a40a46a56a6da8ca9aabaac2aebb08b13b17b3ab42b59ba8bd4be2c14c24c26c34c51"
"c71c8fcb4cd8cded24d45d6ad9bdc3dd1e03e05e07e08e1ae2ae56e60e8aea5eaaec0ecdedbef0f11f21f40f42f54f98";
static void iq3xxs_entry(int idx, int out[4]) {
  int c = 0;
  for (int k = 0; k < 3; ++k) {
    const char ch = iq3xxs_codes[3 * idx + k];
    c = c * 16 + (ch <= '9' ? ch - '0' : ch - 'a' + 10);
  }
  for (int j = 0; j < 4; ++j) {
    const int i = (c >> (3 * j)) & 7;
    out[j] = i == 7 ? 62 : 4 + 8 * i;
  }
}
static void iq3s_entry(int idx, int out[4]) {
  int c = 0;
  for (int k = 0; k < 3; ++k) {
    const char ch = iq3s_codes[3 * idx + k];
    c = c * 16 + (ch <= '9' ? ch - '0' : ch - 'a' + 10);
  }
  for (int j = 0; j < 4; ++j) out[j] = 2 * ((c >> (3 * j)) & 7) + 1;
}

typedef struct {
  float d, dmin;
  int sc[8], mn[8];
  int sc6[16];
  float d8[8];
  int16_t q[256];
} orc_sb;

static uint16_t rd16(const uint8_t* p) { uint16_t v; memcpy(&v, p, 2); return v; }

int orc_decode_sb(uint32_t type, const uint8_t* p, orc_sb* o) {
  memset(o, 0, sizeof *o);
  if (ORC_Q45(type)) {
    o->d = orc_fp16_to_f32(rd16(p));
    o->dmin = orc_fp16_to_f32(rd16(p + 2));
    for (int b = 0; b < 8; ++b) scale_min_k4(b, p + 4, &o->sc[b], &o->mn[b]);
    /* Q5_K: 32 bytes of fifth bits between the scales and the nibbles; bit b of byte l belongs to element 32 b + l */
    const uint8_t* qh = type == ORC_Q5_K ? p + 16 : NULL;
    const uint8_t* qs = type == ORC_Q5_K ? p + 48 : p + 16;
    for (int j = 0; j < 4; ++j)
      for (int l = 0; l < 32; ++l) {
        int lo = qs[32 * j + l] & 0xF, hi = qs[32 * j + l] >> 4;
        if (qh) {
          lo += 16 * ((qh[l] >> (2 * j)) & 1);
          hi += 16 * ((qh[l] >> (2 * j + 1)) & 1);
        }
        o->q[64 * j + l] = (int16_t)lo;
        o->q[64 * j + 32 + l] = (int16_t)hi;
      }
    return 0;
  }
  if (type == ORC_Q6_K) {
    const uint8_t *ql = p, *qh = p + 128;
    const int8_t* sc = (const int8_t*)(p + 192);
    o->d = orc_fp16_to_f32(rd16(p + 208));
    for (int i = 0; i < 16; ++i) o->sc6[i] = sc[i];
    for (int n = 0; n < 2; ++n)
      for (int l = 0; l < 32; ++l) {
        const uint8_t *L = ql + 64 * n, *H = qh + 32 * n;
        o->q[128 * n + l + 0] = (int16_t)((L[l] & 0xF) | (((H[l] >> 0) & 3) << 4));
        o->q[128 * n + l + 32] = (int16_t)((L[l + 32] & 0xF) | (((H[l] >> 2) & 3) << 4));
        o->q[128 * n + l + 64] = (int16_t)((L[l] >> 4) | (((H[l] >> 4) & 3) << 4));
        o->q[128 * n + l + 96] = (int16_t)((L[l + 32] >> 4) | (((H[l] >> 6) & 3) << 4));
      }
    return 0;
  }
  if (type == ORC_IQ4_XS) { /* f16 d, 16 bits of scale high parts, 4 bytes of low nibbles, 8 blocks of 16 bytes: the low
                               nibbles are a block's elements 0..15, the high ones 16..31 */
    o->d = orc_fp16_to_f32(rd16(p));
    const unsigned sh = rd16(p + 2);
    for (int ib = 0; ib < 8; ++ib) {
      const int ls = ((p[4 + ib / 2] >> (4 * (ib % 2))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4);
      o->sc6[2 * ib] = o->sc6[2 * ib + 1] = ls - 32;
      for (int j = 0; j < 16; ++j) {
        o->q[32 * ib + j] = iq4_values[p[8 + 16 * ib + j] & 0xF];
        o->q[32 * ib + 16 + j] = iq4_values[p[8 + 16 * ib + j] >> 4];
      }
    }
    return 0;
  }
  if (type == ORC_IQ3_S) { /* 110 bytes: f16 d, qs[64] (the low 8 bits of a grid index per 4 values), qh[8] (the ninth
                              bits of a 32-block's 8 indices), signs[32] (one bit per value), scales[4] (a nibble per
                              32-block: sub-scale 1 + 2 s); src/quants.h:240-262 */
    o->d = orc_fp16_to_f32(rd16(p));
    const uint8_t *qs = p + 2, *qh = p + 66, *sg = p + 74, *scl = p + 106;
    for (int ib = 0; ib < 8; ++ib) {
      o->sc6[2 * ib] = o->sc6[2 * ib + 1] = 1 + 2 * ((scl[ib / 2] >> (4 * (ib % 2))) & 0xF);
      for (int g = 0; g < 8; ++g) { /* group g of the block: values 4 g .. 4 g + 3 */
        const int idx = qs[8 * ib + g] | (((qh[ib] >> g) & 1) << 8);
        int m[4];
        iq3s_entry(idx, m);
        for (int j = 0; j < 4; ++j) {
          const int e = 4 * g + j; /* sign bit e % 8 of the block's byte e / 8 */
          o->q[32 * ib + e] = (int16_t)(((sg[4 * ib + e / 8] >> (e % 8)) & 1) ? -m[j] : m[j]);
        }
      }
    }
    return 0;
  }
  if (type == ORC_Q8_0) {
    for (int b = 0; b < 8; ++b) {
      const uint8_t* blk = p + 34 * b;
      o->d8[b] = orc_fp16_to_f32(rd16(blk));
      for (int i = 0; i < 32; ++i) o->q[32 * b + i] = (int8_t)blk[2 + i];
    }
    return 0;
  }
  if (type == ORC_IQ3_XXS) { /* 98 bytes: f16 d, qs[64] (a codebook index per 4 values), then per 32-block a word: four
                                7-bit sign codes (code l: the signs of values 8 l .. 8 l + 7, the eighth bit the
                                parity of the seven -- ggml's ksigns_iq2xs) and in the top nibble the scale s;
                                value = d / 4 * (1 + 2 s) * the signed magnitude (src/quants.h:220-239) */
    o->d = orc_fp16_to_f32(rd16(p)) / 4;
    const uint8_t *qs = p + 2, *ss = p + 66;
    for (int ib = 0; ib < 8; ++ib) {
      uint32_t a;
      memcpy(&a, ss + 4 * ib, 4);
      o->sc6[2 * ib] = o->sc6[2 * ib + 1] = 1 + 2 * (int)(a >> 28);
      for (int l = 0; l < 4; ++l) {
        uint32_t sg = (a >> (7 * l)) & 127u, par = sg;
        par ^= par >> 4; par ^= par >> 2; par ^= par >> 1;
        sg |= (par & 1u) << 7;
        for (int h = 0; h < 2; ++h) {
          int m[4];
          iq3xxs_entry(qs[8 * ib + 2 * l + h], m);
          for (int j = 0; j < 4; ++j)
            o->q[32 * ib + 8 * l + 4 * h + j] = (int16_t)(((sg >> (4 * h + j)) & 1) ? -m[j] : m[j]);
        }
      }
    }
    return 0;
  }
  if (type == ORC_Q3_K) { /* 110 bytes: hmask[32] (bit b of byte e: the third bit of element e of 32-block b), qs[64]
                             (two bits of element e of block b: byte 32 (b / 4) + e, bits 2 (b % 4)), 12 bytes of sixteen
                             6-bit scales (scale i: low nibble i / 8 of byte i % 8, top two bits: bits 2 (i / 4) of byte
                             8 + i % 4), f16 d; value = d * (scale - 32) * (q - 4), q the three bits
                             (src/quants.h:465-494) */
    const uint8_t *hm = p, *qs = p + 32, *sc = p + 96;
    o->d = orc_fp16_to_f32(rd16(p + 108));
    for (int i = 0; i < 16; ++i)
      o->sc6[i] = (int)(((sc[i & 7] >> (4 * (i >> 3))) & 0xF) | (((sc[8 + (i & 3)] >> (2 * (i >> 2))) & 3) << 4)) - 32;
    for (int b = 0; b < 8; ++b)
      for (int e = 0; e < 32; ++e)
        o->q[32 * b + e] = (int16_t)(((qs[32 * (b / 4) + e] >> (2 * (b % 4))) & 3) + (((hm[e] >> b) & 1) ? 4 : 0) - 4);
    return 0;
  }
  if (type == ORC_IQ4_NL) { /* 8 blocks of 18 bytes: f16 d, low nibbles = elements 0..15, high = 16..31, each a code of
                               the IQ4 table (src/quants.h:594-606) */
    for (int b = 0; b < 8; ++b) {
      const uint8_t* blk = p + 18 * b;
      o->d8[b] = orc_fp16_to_f32(rd16(blk));
      for (int i = 0; i < 16; ++i) {
        o->q[32 * b + i] = iq4_values[blk[2 + i] & 0xF];
        o->q[32 * b + 16 + i] = iq4_values[blk[2 + i] >> 4];
      }
    }
    return 0;
  }
  if (type == ORC_MXFP4) { /* 8 blocks of 17 bytes: E8M0 scale byte e, then the nibbles as above, each an E2M1 code whose
                              doubled value is in the table; value = 2^(e - 128) * table[code] (src/quants.h:495-503,
                              520-530; e = 0 and 1 give the f32 subnormals 2^-128 and 2^-127) */
    static const int8_t mxfp4_values[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
    for (int b = 0; b < 8; ++b) {
      const uint8_t* blk = p + 17 * b;
      const uint32_t bits = blk[0] < 2 ? 0x00200000u << blk[0] : (uint32_t)(blk[0] - 1) << 23;
      memcpy(&o->d8[b], &bits, 4);
      for (int i = 0; i < 16; ++i) {
        o->q[32 * b + i] = mxfp4_values[blk[1 + i] & 0xF];
        o->q[32 * b + 16 + i] = mxfp4_values[blk[1 + i] >> 4];
      }
    }
    return 0;
  }
  if (type == ORC_AR4_128) { /* 2 blocks of 66 bytes: f16 d, then four runs of 16 bytes, each the nibbles of 32 elements
                                as Q4_0 holds them, q - 8 (src/quants.h:531-542) */
    for (int b = 0; b < 8; ++b) {
      const uint8_t* blk = p + 66 * (b / 4);
      o->d8[b] = orc_fp16_to_f32(rd16(blk));
      for (int i = 0; i < 16; ++i) {
        o->q[32 * b + i] = (int16_t)((blk[2 + 16 * (b % 4) + i] & 0xF) - 8);
        o->q[32 * b + 16 + i] = (int16_t)((blk[2 + 16 * (b % 4) + i] >> 4) - 8);
      }
    }
    return 0;
  }
  if (type == ORC_Q2_0) { /* 4 blocks of 18 bytes: f16 d, then 64 2-bit codes, element j in bits 2 (j % 4) of byte j / 4,
                             q - 1 (src/quants.h:607-616) */
    for (int b = 0; b < 8; ++b) {
      const uint8_t* blk = p + 18 * (b / 2);
      o->d8[b] = orc_fp16_to_f32(rd16(blk));
      for (int i = 0; i < 32; ++i) {
        const int j = 32 * (b % 2) + i;
        o->q[32 * b + i] = (int16_t)(((blk[2 + j / 4] >> (2 * (j % 4))) & 3) - 1);
      }
    }
    return 0;
  }
  if (type == ORC_Q4_0) { /* 8 blocks of 18 bytes: f16 d, low nibbles = elements 0..15, high = 16..31, q - 8
                             (src/quants.h:136-148) */
    for (int b = 0; b < 8; ++b) {
      const uint8_t* blk = p + 18 * b;
      o->d8[b] = orc_fp16_to_f32(rd16(blk));
      for (int i = 0; i < 16; ++i) {
        o->q[32 * b + i] = (int16_t)((blk[2 + i] & 0xF) - 8);
        o->q[32 * b + 16 + i] = (int16_t)((blk[2 + i] >> 4) - 8);
      }
    }
    return 0;
  }
  return -1;
}

/* Value of element e of a decoded superblock, f32, evaluated left to right as written (src/quants.h:317-324). */
static float sb_value(uint32_t type, const orc_sb* o, int e) {
  if (ORC_Q45(type)) return o->d * (float)o->sc[e / 32] * (float)o->q[e] - o->dmin * (float)o->mn[e / 32];
  if (type == ORC_Q6_K) return o->d * (float)o->sc6[e / 16] * (float)(o->q[e] - 32);
  if (ORC_IQLIKE(type)) return o->d * (float)o->sc6[e / 16] * (float)o->q[e]; /* (src/quants.h:321-323 generic: wd * wsc * q) */
  return o->d8[e / 32] * (float)o->q[e];
}

/* The signed integer the int8 dot product sees for element e: Q4_K q (0..15), Q6_K q - 32, Q8_0 q
 * (zero/kernels/decode.cl:221-260). */
static int sb_int(uint32_t type, const orc_sb* o, int e) { return type == ORC_Q6_K ? o->q[e] - 32 : o->q[e]; }

/* One row of K elements to f32 (src/quants.h:519, generic tail 617-621).  K % 256 == 0. */
int orc_dequant_row(uint32_t type, const uint8_t* row, int K, float* out) {
  const int bb = orc_sb_bytes(type);
  if (!bb || K % 256) return -1;
  orc_sb o;
  for (int s = 0; s < K / 256; ++s) {
    orc_decode_sb(type, row + (size_t)s * bb, &o);
    for (int e = 0; e < 256; ++e) out[s * 256 + e] = sb_value(type, &o, e);
  }
  return 0;
}

/* Decoded integer fields of one row, for tests: q [K] (as the dot product sees them), isc [K/16] integer sub-scale
 * per 16 elements (Q4_K: the block's 6-bit scale twice, Q6_K: the int8 scales, Q8_0: 1), imn [K/16] (Q4_K mins twice,
 * else 0), d [K/32] f32 scale per 32-block (Q4_K / Q6_K: the superblock's d repeated), dmin [K/32]. */
int orc_decode_row_fields(uint32_t type, const uint8_t* row, int K, int8_t* q, int32_t* isc, int32_t* imn, float* d,
                          float* dmin) {
  const int bb = orc_sb_bytes(type);
  if (!bb || K % 256) return -1;
  orc_sb o;
  for (int s = 0; s < K / 256; ++s) {
    orc_decode_sb(type, row + (size_t)s * bb, &o);
    for (int e = 0; e < 256; ++e) q[s * 256 + e] = (int8_t)sb_int(type, &o, e);
    for (int h = 0; h < 16; ++h) {
      isc[s * 16 + h] = ORC_Q45(type) ? o.sc[h / 2] : ORC_Q6LIKE(type) ? o.sc6[h] : 1;
      imn[s * 16 + h] = ORC_Q45(type) ? o.mn[h / 2] : 0;
    }
    for (int b = 0; b < 8; ++b) {
      d[s * 8 + b] = ORC_Q8LIKE(type) ? o.d8[b] : o.d;
      dmin[s * 8 + b] = ORC_Q45(type) ? o.dmin : 0.0f;
    }
  }
  return 0;
}

/* ---------------------------------------------------------------- quantizers */

/* Activation quantizer: int8 per block of 32 (act32) or 256 with an absmax scale, and the int16 sum of every 16
 * int8 values.  aq [M][K], asc [K/B][M], absum [K/16][M]  (src/quants.h:626-643 == zero/kernels/ops.cl:38-72).
 * inv = 127/amax, q = lrintf(v * inv) under round-to-nearest-even, scale = amax / 127. */
void orc_quantize_act(const float* x, int M, int K, int8_t* aq, float* asc, int16_t* absum, int act32) {
  const int B = act32 ? 32 : 256;
  for (int m = 0; m < M; ++m)
    for (int b0 = 0; b0 < K; b0 += B) {
      const float* v = x + (size_t)m * K + b0;
      float amax = 0;
      for (int i = 0; i < B; ++i) amax = fmaxf(amax, fabsf(v[i]));
      const float inv = amax > 0 ? 127.0f / amax : 0.0f;
      asc[(size_t)(b0 / B) * M + m] = amax / 127.0f;
      for (int i = 0; i < B; ++i) {
        const float p = v[i] * inv; /* one f32 multiply, no fma */
        aq[(size_t)m * K + b0 + i] = (int8_t)lrintf(p);
      }
    }
  for (int m = 0; m < M; ++m)
    for (int b = 0; b < K / 16; ++b) {
      int sum = 0;
      for (int i = 0; i < 16; ++i) sum += aq[(size_t)m * K + b * 16 + i];
      absum[(size_t)b * M + m] = (int16_t)sum;
    }
}

/* What the int8 values miss, for the two-pass matmul inputs (zero/kernels/ops.cl:49-59): res = v - (float)q * (amax / 127)
 * per element, the product and the difference each rounded to f32 (this file is built without contraction; the
 * reference's OpenCL text leaves that to its compiler).  res [M][K]; quantized by orc_quantize_act it gives the second
 * pass's inputs (ops.cl:73-101).  PARITY UNPINNED against a run of the reference (its CPU twin quantize_act_cpu has no
 * residual and no test vector holds one); pinned by what the mathematics fixes: q * scale + res == v exactly whenever
 * the subtraction is exact (Sterbenz: always, here, for q != 0 -- see the tests), and |res| <= scale / 2 (1 + 2^-22). */
void orc_act_residual(const float* x, int M, int K, const int8_t* aq, const float* asc, int act32, float* res) {
  const int B = act32 ? 32 : 256;
  for (int m = 0; m < M; ++m)
    for (int e = 0; e < K; ++e) {
      const float sc = asc[(size_t)(e / B) * M + m];
      const float p = (float)aq[(size_t)m * K + e] * sc;
      res[(size_t)m * K + e] = x[(size_t)m * K + e] - p;
    }
}

/* The expert input quantizer (zero/kernels/moe.cl:258-274): as orc_quantize_act with act32, rows of F values, scales
 * hsc [(F/32)][S] with row stride S (the slot count), no sums. */
void orc_moe_quant(const float* h, int n, int F, int S, int8_t* hq, float* hsc) {
  for (int r = 0; r < n; ++r)
    for (int b = 0; b < F / 32; ++b) {
      const float* v = h + (size_t)r * F + 32 * b;
      float amax = 0;
      for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
      const float inv = amax > 0 ? 127.0f / amax : 0.0f;
      hsc[(size_t)b * S + r] = amax / 127.0f;
      for (int i = 0; i < 32; ++i) {
        const float p = v[i] * inv;
        hq[(size_t)r * F + 32 * b + i] = (int8_t)lrintf(p);
      }
    }
}

/* f32 rows [N][K] -> GGUF Q8_0 blocks: d = amax / 127 (stored as fp16 of that f32), q = lrintf(v * (1 / d)) with the
 * f32 d, not the rounded one (src/quants.h:429-442). out: N * K/32 * 34 bytes. */
void orc_quantize_rows_q8_0(const float* src, int N, int K, uint8_t* out) {
  for (size_t b = 0; b < (size_t)N * (size_t)(K / 32); ++b) {
    const float* v = src + b * 32;
    float amax = 0;
    for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
    const float d = amax / 127.0f, inv = d > 0 ? 1.0f / d : 0.0f;
    uint8_t* blk = out + b * 34;
    const uint16_t dh = orc_f32_to_fp16(d);
    memcpy(blk, &dh, 2);
    for (int i = 0; i < 32; ++i) {
      const float p = v[i] * inv;
      blk[2 + i] = (uint8_t)(int8_t)lrintf(p);
    }
  }
}

/* f32 rows [N][K] -> GGUF Q4_0 blocks as llama.cpp's quantize_row_q4_0_ref: d = (the value of largest magnitude) / -8,
 * q = min(15, (int)(v / d + 8.5)), element i in the low nibble of byte i, element i + 16 in the high
 * (src/quants.h:444-463). out: N * K/32 * 18 bytes. */
void orc_quantize_rows_q4_0(const float* src, int N, int K, uint8_t* out) {
  for (size_t b = 0; b < (size_t)N * (size_t)(K / 32); ++b) {
    const float* v = src + b * 32;
    float amax = 0, mx = 0;
    for (int i = 0; i < 32; ++i)
      if (fabsf(v[i]) > amax) { amax = fabsf(v[i]); mx = v[i]; }
    const float d = mx / -8.0f, id = d != 0 ? 1.0f / d : 0.0f;
    uint8_t* blk = out + b * 18;
    const uint16_t dh = orc_f32_to_fp16(d);
    memcpy(blk, &dh, 2);
    for (int i = 0; i < 16; ++i) {
      int q0 = (int)(v[i] * id + 8.5f), q1 = (int)(v[i + 16] * id + 8.5f);
      if (q0 > 15) q0 = 15;
      if (q1 > 15) q1 = 15;
      blk[2 + i] = (uint8_t)(q0 | (q1 << 4));
    }
  }
}

/* ---------------------------------------------------------------- integer block sums */

/* I [M][N][K/16]: the int32 dot product of every 16-element half block of weight row n with token row m
 * (zero/kernels/decode.cl:992-999: lo / hi).  A 32-block's sum is the sum of its two halves. */
int orc_block_sums(uint32_t type, const uint8_t* W, int N, int K, const int8_t* aq, int M, int32_t* I) {
  const int bb = orc_sb_bytes(type), nsb = K / 256;
  if (!bb || K % 256) return -1;
#pragma omp parallel for schedule(dynamic, 16)
  for (int n = 0; n < N; ++n) {
    orc_sb o;
    for (int s = 0; s < nsb; ++s) {
      orc_decode_sb(type, W + ((size_t)n * nsb + s) * bb, &o);
      for (int m = 0; m < M; ++m)
        for (int h = 0; h < 16; ++h) {
          int32_t acc = 0;
          for (int i = 0; i < 16; ++i) acc += sb_int(type, &o, 16 * h + i) * (int32_t)aq[(size_t)m * K + s * 256 + 16 * h + i];
          I[((size_t)m * N + n) * (K / 16) + s * 16 + h] = acc;
        }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------- f32 references */

/* Y[m][n] = (float) sum_k (double)dequant(W)[n][k] * (double)((float)aq[m][k] * asc[k/32][m]): the reference's CPU
 * matmul (tools/ref_forward.cpp:268-303: OpenMP over output rows, schedule(dynamic, 16), dequant_row once per row,
 * double-accumulated dot per token) on activations rounded as the engine rounds them
 * (tools/ref_forward.cpp:109-126 round_int8 with B = 32; bench/gemv_bench.cpp:121-123, 203-207: xq = q * sc).
 * asc has row stride Ms (>= M).  Y row stride ldy. */
int orc_matmul_ref(uint32_t type, const uint8_t* W, int N, int K, const int8_t* aq, const float* asc, int Ms, int M,
                   float* Y, int ldy) {
  const int bb = orc_sb_bytes(type), nsb = K / 256;
  if (!bb || K % 256) return -1;
  float* X = (float*)malloc((size_t)M * K * sizeof(float));
  if (!X) return -2;
  for (int m = 0; m < M; ++m)
    for (int k = 0; k < K; ++k) X[(size_t)m * K + k] = (float)aq[(size_t)m * K + k] * asc[(size_t)(k / 32) * Ms + m];
#pragma omp parallel
  {
    float* w = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(dynamic, 16)
    for (int n = 0; n < N; ++n) {
      orc_dequant_row(type, W + (size_t)n * nsb * bb, K, w);
      for (int m = 0; m < M; ++m) {
        double acc = 0;
        const float* x = X + (size_t)m * K;
        for (int k = 0; k < K; ++k) acc += (double)w[k] * x[k];
        Y[(size_t)m * ldy + n] = (float)acc;
      }
    }
    free(w);
  }
  free(X);
  return 0;
}

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* The engine's own arithmetic, in f32, from the integer block sums.
 *   form 0 (GEMV, zero/kernels/decode.cl:1000-1003), per 32-block b in order:
 *     Q4_K: acc += sa * (d * (float)(sc*lo + sc*hi) - dmin * (float)(mn*bs0 + mn*bs1))
 *     Q6_K / Q8_0: acc += sa * d * (float)(sc0*lo + sc1*hi)
 *   form 1 (GEMM with per-32 activation scales, zero/kernels/gemm.cl:439-488), per superblock, block pairs (2j, 2j+1):
 *     Q4_K: tq = fma(avl,(float)plo, fma(avh,(float)phi,tq)); tmn likewise; res = fma(d,tq, fma(-dmin,tmn,res))
 *     Q6_K: plo = acc0*sc0 + acc1*sc1; tq as above; res = fma(d,tq,res)
 *     Q8_0: res = fma(avl*dlo,(float)acc0, fma(avh*dhi,(float)acc1,res))
 * The reference's lanes add their partial sums in an implementation-defined tree (sub_group_reduce_add); this
 * restatement adds in block order, so it is a second f32 evaluation to compare within rounding, not bit for bit. */
int orc_matmul_formula(uint32_t type, int form, const uint8_t* W, int N, int K, const int8_t* aq, const float* asc,
                       const int16_t* absum, int Ms, int M, float* Y, int ldy) {
  const int bb = orc_sb_bytes(type), nsb = K / 256;
  if (!bb || K % 256) return -1;
#pragma omp parallel for schedule(dynamic, 16)
  for (int n = 0; n < N; ++n) {
    orc_sb o;
    for (int m = 0; m < M; ++m) {
      float res = 0.0f;
      for (int s = 0; s < nsb; ++s) {
        orc_decode_sb(type, W + ((size_t)n * nsb + s) * bb, &o);
        int32_t h16[16];
        for (int h = 0; h < 16; ++h) {
          int32_t acc = 0;
          for (int i = 0; i < 16; ++i) acc += sb_int(type, &o, 16 * h + i) * (int32_t)aq[(size_t)m * K + s * 256 + 16 * h + i];
          h16[h] = acc;
        }
        float tq = 0.0f, tmn = 0.0f;
        for (int j = 0; j < 4; ++j) {
          float t2[2], m2[2], sa2[2];
          for (int u = 0; u < 2; ++u) {
            const int b = 2 * j + u;
            const float sa = asc[(size_t)(s * 8 + b) * Ms + m];
            const int lo = h16[2 * b], hi = h16[2 * b + 1];
            const int bs0 = absum[(size_t)(s * 16 + 2 * b) * Ms + m], bs1 = absum[(size_t)(s * 16 + 2 * b + 1) * Ms + m];
            sa2[u] = sa;
            if (ORC_Q45(type)) {
              t2[u] = (float)(o.sc[b] * lo + o.sc[b] * hi);
              m2[u] = (float)(o.mn[b] * bs0 + o.mn[b] * bs1);
              if (form == 0) res += sa * (o.d * t2[u] - o.dmin * m2[u]);
            } else if (ORC_Q6LIKE(type)) {
              t2[u] = (float)(o.sc6[2 * b] * lo + o.sc6[2 * b + 1] * hi);
              m2[u] = 0.0f;
              if (form == 0) res += sa * o.d * t2[u];
            } else {
              t2[u] = (float)(lo + hi);
              m2[u] = 0.0f;
              if (form == 0) res += sa * o.d8[b] * t2[u];
            }
          }
          if (form == 1) {
            if (ORC_Q8LIKE(type)) {
              res = fmaf(sa2[0] * o.d8[2 * j], t2[0], fmaf(sa2[1] * o.d8[2 * j + 1], t2[1], res));
            } else {
              tq = fmaf(sa2[0], t2[0], fmaf(sa2[1], t2[1], tq));
              tmn = fmaf(sa2[0], m2[0], fmaf(sa2[1], m2[1], tmn));
            }
          }
        }
        if (form == 1 && ORC_Q45(type)) res = fmaf(o.d, tq, fmaf(-o.dmin, tmn, res));
        if (form == 1 && ORC_Q6LIKE(type)) res = fmaf(o.d, tq, res);
      }
      Y[(size_t)m * ldy + n] = res;
    }
  }
  return 0;
}

/* ---------------------------------------------------------------- mixture of experts */

/* silu as the CPU reference evaluates it (tools/ref_forward.cpp:321): below -80 the result is 0. */
float orc_silu(float x) { return x < -80.0f ? 0.0f : x / (1.0f + expf(-x)); }

/* Routing of T tokens (zero/kernels/moe.cl:50-89): the NU largest of NE logits (ties: the lower expert id),
 * p_k = exp(l_k - max l), weights p_k / sum of the selected p; per-expert counts; sgate = sigmoid(l[NE]) when the
 * row has a shared-expert logit at column NE (ldl > NE), else 0.5 is NOT written: sgate may be NULL. */
/* The routing variants of zero/kernels/moe.cl:17-46 (parity unpinned: none of the reference's tests or files holds a
 * vector of them; held by a float64 numpy restatement of the same formulas in tests/test_gpu_moe.py): escale (-DESCALE):
 * the weight times escale[e] after the normalization; ebias + rscale (-DROUTE_DS -DRSCALE): score s = sqrt(softplus(l)),
 * chosen by s + ebias[e], weight s / (sum + 1e-20) * rscale, shared-expert gate 1. */
static float orc_ds_sp(float g) { return sqrtf(g > 20.0f ? g + log1pf(expf(-g)) : log1pf(expf(g))); }
void orc_moe_route_v(const float* logits, int ldl, int T, int NE, int NU, int32_t* ids, float* wts, float* sgate,
                     int32_t* counts, const float* escale, const float* ebias, float rscale) {
  for (int e = 0; e < NE; ++e) counts[e] = 0;
  float* v = (float*)malloc((size_t)NE * sizeof(float));
  for (int t = 0; t < T; ++t) {
    const float* lg = logits + (size_t)t * ldl;
    float mx = -INFINITY;
    for (int e = 0; e < NE; ++e) { v[e] = ebias ? orc_ds_sp(lg[e]) + ebias[e] : lg[e]; mx = fmaxf(mx, v[e]); }
    float p[64], sum = 0.0f;
    int sel[64];
    for (int k = 0; k < NU; ++k) {
      float bv = -INFINITY;
      int bi = NE;
      for (int e = 0; e < NE; ++e)
        if (v[e] > bv) { bv = v[e]; bi = e; }
      if (bi < NE) v[bi] = -INFINITY;
      sel[k] = bi < NE - 1 ? bi : NE - 1;
      p[k] = ebias ? orc_ds_sp(lg[sel[k]]) : expf(bv - mx);
      sum += p[k];
    }
    for (int k = 0; k < NU; ++k) {
      float w = ebias ? p[k] / (sum + 1e-20f) * rscale : p[k] / sum;
      if (escale) w *= escale[sel[k]];
      ids[(size_t)t * NU + k] = sel[k];
      wts[(size_t)t * NU + k] = w;
      counts[sel[k]]++;
    }
    if (sgate) sgate[t] = ebias ? 1.0f : ldl > NE ? 1.0f / (1.0f + expf(-lg[NE])) : 0.0f;
  }
  free(v);
}

void orc_moe_route(const float* logits, int ldl, int T, int NE, int NU, int32_t* ids, float* wts, float* sgate,
                   int32_t* counts) {
  for (int e = 0; e < NE; ++e) counts[e] = 0;
  float* v = (float*)malloc((size_t)NE * sizeof(float));
  for (int t = 0; t < T; ++t) {
    const float* lg = logits + (size_t)t * ldl;
    float mx = -INFINITY;
    for (int e = 0; e < NE; ++e) { v[e] = lg[e]; mx = fmaxf(mx, v[e]); }
    float p[64], sum = 0.0f;
    int sel[64];
    for (int k = 0; k < NU; ++k) {
      float bv = -INFINITY;
      int bi = NE;
      for (int e = 0; e < NE; ++e)
        if (v[e] > bv) { bv = v[e]; bi = e; } /* strict >: the lowest index of equal values wins */
      if (bi < NE) v[bi] = -INFINITY;
      sel[k] = bi < NE - 1 ? bi : NE - 1; /* (a row of NaN picks nothing: clamped as moe.cl:77) */
      p[k] = expf(bv - mx);
      sum += p[k];
    }
    for (int k = 0; k < NU; ++k) {
      ids[(size_t)t * NU + k] = sel[k];
      wts[(size_t)t * NU + k] = p[k] / sum;
      counts[sel[k]]++;
    }
    if (sgate) sgate[t] = ldl > NE ? 1.0f / (1.0f + expf(-lg[NE])) : 0.0f;
  }
  free(v);
}

/* Exclusive scan of the counts and the tile list (zero/kernels/moe.cl:141-168): offs[e], tstart[e] (first tile of
 * expert e), tstart[NE] = tile count, tiles[0] = tile count then (expert, first slot, rows <= TM) per tile. */
void orc_moe_scan(const int32_t* counts, int NE, int TM, int32_t* offs, int32_t* tiles, int32_t* tstart) {
  int off = 0, toff = 0;
  for (int e = 0; e < NE; ++e) {
    const int c = counts[e], nt = (c + TM - 1) / TM;
    offs[e] = off;
    tstart[e] = toff;
    for (int i = 0; i < nt; ++i) {
      tiles[1 + 3 * (toff + i) + 0] = e;
      tiles[1 + 3 * (toff + i) + 1] = off + i * TM;
      tiles[1 + 3 * (toff + i) + 2] = c - i * TM < TM ? c - i * TM : TM;
    }
    off += c;
    toff += nt;
  }
  tiles[0] = tstart[NE] = toff;
}

/* Slots in pair order (zero/kernels/moe.cl:171-179 with its atomic counter replaced by the serial order; the
 * reference's slot order inside an expert is not deterministic, its results are). */
void orc_moe_scatter(const int32_t* ids, const float* wts, int n, int NU, const int32_t* offs, int NE, int32_t* stok,
                     float* swt, int32_t* inv) {
  int32_t* cur = (int32_t*)malloc((size_t)NE * sizeof(int32_t));
  memcpy(cur, offs, (size_t)NE * sizeof(int32_t));
  for (int i = 0; i < n; ++i) {
    const int s = cur[ids[i]]++;
    stok[s] = i / NU;
    swt[s] = wts[i];
    inv[i] = s;
  }
  free(cur);
}

/* One MoE FFN over T tokens (zero/engine_moe.h:8-361 with standard expert tensors and no shared expert;
 * tools/ref_forward.cpp:333-364 expert_mv per (token, expert)):
 *   route -> per pair: g = Wg_e x, u = Wu_e x (x = the token's int8-rounded input), h = silu(g) * u,
 *   h rounded to int8 per 32 (zero/kernels/moe.cl:258-274), v = Wd_e h, y = w * v; out[t] = sum_k y (k order,
 *   zero/kernels/moe.cl:349-351).
 * Dot products as orc_matmul_ref (double accumulation of dequantized weights).  The gate / up sums are rounded to
 * f32 before the SwiGLU, as the engine stores them.  Wg, Wu: [NE][F][E] rows, Wd: [NE][E][F] rows, GGUF blocks.
 * Also returns h [T*NU][F] (pair order) when h_out is not NULL. */
int orc_moe_layer(uint32_t type, const uint8_t* Wg, const uint8_t* Wu, const uint8_t* Wd, int NE, int NU, int E, int F,
                  const int8_t* aq, const float* asc, int Ms, int T, const float* logits, int ldl, float* out,
                  float* h_out) {
  const int bb = orc_sb_bytes(type);
  if (!bb || E % 256 || F % 256) return -1;
  const size_t rbE = (size_t)(E / 256) * bb, rbF = (size_t)(F / 256) * bb;
  int32_t* ids = (int32_t*)malloc((size_t)T * NU * 4);
  float* wts = (float*)malloc((size_t)T * NU * 4);
  int32_t* counts = (int32_t*)malloc((size_t)NE * 4);
  orc_moe_route(logits, ldl, T, NE, NU, ids, wts, NULL, counts);
  memset(out, 0, (size_t)T * E * sizeof(float));
  float* Y = (float*)malloc((size_t)T * NU * E * sizeof(float));
#pragma omp parallel
  {
    float* w = (float*)malloc((size_t)(E > F ? E : F) * sizeof(float));
    float* x = (float*)malloc((size_t)E * sizeof(float));
    float* h = (float*)malloc((size_t)F * sizeof(float));
    int8_t* hq = (int8_t*)malloc((size_t)F);
    float* hs = (float*)malloc((size_t)(F / 32) * sizeof(float));
    float* hx = (float*)malloc((size_t)F * sizeof(float));
#pragma omp for schedule(dynamic, 4)
    for (int i = 0; i < T * NU; ++i) {
      const int t = i / NU, e = ids[i];
      for (int k = 0; k < E; ++k) x[k] = (float)aq[(size_t)t * E + k] * asc[(size_t)(k / 32) * Ms + t];
      for (int f = 0; f < F; ++f) {
        double g = 0, u = 0;
        orc_dequant_row(type, Wg + ((size_t)e * F + f) * rbE, E, w);
        for (int k = 0; k < E; ++k) g += (double)w[k] * x[k];
        orc_dequant_row(type, Wu + ((size_t)e * F + f) * rbE, E, w);
        for (int k = 0; k < E; ++k) u += (double)w[k] * x[k];
        h[f] = orc_silu((float)g) * (float)u;
      }
      if (h_out) memcpy(h_out + (size_t)i * F, h, (size_t)F * sizeof(float));
      orc_moe_quant(h, 1, F, 1, hq, hs);
      for (int f = 0; f < F; ++f) hx[f] = (float)hq[f] * hs[f / 32];
      for (int c = 0; c < E; ++c) {
        double v = 0;
        orc_dequant_row(type, Wd + ((size_t)e * E + c) * rbF, F, w);
        for (int f = 0; f < F; ++f) v += (double)w[f] * hx[f];
        Y[(size_t)i * E + c] = wts[i] * (float)v;
      }
    }
    free(w); free(x); free(h); free(hq); free(hs); free(hx);
  }
  for (int t = 0; t < T; ++t)
    for (int c = 0; c < E; ++c) {
      float v = 0.0f;
      for (int k = 0; k < NU; ++k) v += Y[((size_t)t * NU + k) * E + c];
      out[(size_t)t * E + c] += v;
    }
  free(ids); free(wts); free(counts); free(Y);
  return 0;
}
