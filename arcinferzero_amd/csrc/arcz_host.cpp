// Host-side helpers of the library that need no GPU: the regrouping of GGUF rows into the device planes (the place of
// the reference's gpu_raw_sb / upload_padded, src/quants.h:728-761, zero/engine_load.h:84-130), the f32 -> Q8_0 row
// quantizer the reference uses for small f32 matrices (src/quants.h:429-442), and the seeded generators of synthetic
// tensors (weights ~ N(0, 0.02) quantized to Q4_K / Q6_K / Q8_0, activations ~ N(0, 1)) that the benchmark and the
// tests share.  The Q4_K / Q6_K quantizers have no counterpart in the reference (it only reads those types): they
// make valid blocks from random values and are input generators, not part of the compute path.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "kernels/common.h"
#define GGML_TYPE_Q4_0 2u  // (GGUF type id, src/gguf.h:19)
#define GGML_TYPE_IQ3_S 21u  // (src/gguf.h:22)
#define GGML_TYPE_IQ4_NL 20u  // (src/gguf.h:21)
#define GGML_TYPE_Q3_K 11u  // (src/gguf.h:20)
#define GGML_TYPE_IQ3_XXS 18u  // (src/gguf.h:21)
#define GGML_TYPE_MXFP4 39u  // (src/gguf.h:23)
#define GGML_TYPE_Q2_0 42u   // (src/gguf.h:30)
#define GGML_TYPE_AR4_128 0x41523447u  // (src/gguf.h:29)

namespace {

// The IQ3_S codebook (ggml's iq3s_grid, a constant of the GGUF format; the reference carries it as src/iq_tables.h:297):
// 512 groups of four magnitudes, each one of 1, 3, ..., 15, here as three hex digits per entry: magnitude j of an entry
// = 2 * ((code >> 3 j) & 7) + 1.
const char kIq3sCodes[] =
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
struct Iq3sGrid {
  uint8_t m[512][4];
  Iq3sGrid() {
    for (int i = 0; i < 512; ++i) {
      int c = 0;
      for (int k = 0; k < 3; ++k) {
        const char ch = kIq3sCodes[3 * i + k];
        c = c * 16 + (ch <= '9' ? ch - '0' : ch - 'a' + 10);
      }
      for (int j = 0; j < 4; ++j) m[i][j] = (uint8_t)(2 * ((c >> (3 * j)) & 7) + 1);
    }
  }
};
const Iq3sGrid kIq3s;

// The IQ3_XXS codebook (ggml's iq3xxs_grid, a constant of the GGUF format; the reference carries it in src/iq_tables.h):
// 256 entries of four magnitudes out of 4, 12, ..., 52, 62, three hex digits an entry, magnitude j its bits 3 j .. 3 j + 2
// as an index into that list.
const char kIq3xxsCodes[] =
"00000200400900b00f01001201902203b03d04104304804a05105505805a06106c07808008208408909009209909b09f"
"0a90af0bd0c10c70c80ca0d50f810b11f12412f13b13d14114715a16a19d1b41c81cc1ce1e31f120120320820a211213"
"21821a21c22722824024224925025228128328828a2912982ba2c02c22d02d92e62f63013053283503543663793853d2"
"3e040040240940b41041241641942244144344544844a45145847347747848048248948f49049249f4a04ad4c14c84cc"
"4f84fc51d52b54355756157c5c15c35ce5e560160860a61161362863563a6406426506596646666816836886956aa6ba"
"6c96db71872773a74074675276d78c79e7b37db7f080480f81d81f82b82f87c89089f8a08b08b68c78e5904929934955"
"9639789c59c89ca9d8a0aa21a38a40a46a56a6da8ca9aabaac2aebb08b13b17b3ab42b59ba8bd4be2c14c24c26c34c51"
"c71c8fcb4cd8cded24d45d6ad9bdc3dd1e03e05e07e08e1ae2ae56e60e8aea5eaaec0ecdedbef0f11f21f40f42f54f98";
struct Iq3xxsGrid {
  uint8_t m[256][4];
  Iq3xxsGrid() {
    for (int i = 0; i < 256; ++i) {
      int c = 0;
      for (int k = 0; k < 3; ++k) {
        const char ch = kIq3xxsCodes[3 * i + k];
        c = c * 16 + (ch <= '9' ? ch - '0' : ch - 'a' + 10);
      }
      for (int j = 0; j < 4; ++j) {
        const int x = (c >> (3 * j)) & 7;
        m[i][j] = (uint8_t)(x == 7 ? 62 : 4 + 8 * x);
      }
    }
  }
};
const Iq3xxsGrid kIq3xxs;

// 256 six-bit values (0..63) into the ql / qh bytes of a Q6_K superblock (reference src/quants.h:115-134 read backwards)
void q6k_pack(const int* q, uint8_t* ql, uint8_t* qh) {
  for (int n = 0; n < 2; ++n)
    for (int l = 0; l < 32; ++l) {
      const int q0 = q[128 * n + l], q1 = q[128 * n + l + 32], q2 = q[128 * n + l + 64], q3 = q[128 * n + l + 96];
      ql[64 * n + l] = (uint8_t)((q0 & 0xF) | ((q2 & 0xF) << 4));
      ql[64 * n + l + 32] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
      qh[32 * n + l] = (uint8_t)((q0 >> 4) | ((q1 >> 4) << 2) | ((q2 >> 4) << 4) | ((q3 >> 4) << 6));
    }
}

// IEEE binary16 conversions, round to nearest even, subnormals kept (the reference's own are src/quants.h:17-52)
float f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu, bits;
  if (e == 0) {
    if (m == 0) bits = sign;
    else {
      int ex = 113;
      while (!(m & 0x400u)) { m <<= 1; --ex; }
      bits = sign | ((uint32_t)ex << 23) | ((m & 0x3FFu) << 13);
    }
  } else if (e == 31) bits = sign | 0x7F800000u | (m << 13);
  else bits = sign | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
uint16_t f32_to_f16(float x) {
  uint32_t f;
  memcpy(&f, &x, 4);
  const uint32_t sign = (f >> 16) & 0x8000u, e8 = (f >> 23) & 0xFFu;
  uint32_t mant = f & 0x7FFFFFu;
  const int e = (int)e8 - 112;
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

inline uint64_t splitmix64(uint64_t& s) {
  uint64_t z = (s += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

}  // namespace

extern "C" {

size_t arcz_gguf_bytes(uint32_t type, size_t rows, int K) {
  const size_t u = rows * (size_t)(K / 256);
  return type == QT_Q4_K ? u * 144 : type == QT_Q5_K ? u * 176 : type == QT_Q6_K ? u * 210 : type == QT_Q8_0 ? u * 272 : type == GGML_TYPE_Q4_0 ? u * 144 : type == QT_IQ4_XS ? u * 136 : type == GGML_TYPE_IQ3_S ? u * 110
         : type == GGML_TYPE_IQ4_NL ? u * 144 : type == GGML_TYPE_MXFP4 ? u * 136 : type == GGML_TYPE_Q3_K ? u * 110 : type == GGML_TYPE_IQ3_XXS ? u * 98 : 0;
}
size_t arcz_planes_bytes(uint32_t type, size_t rows, int K) { return raw_planes_bytes((int)type, rows, K / 256); }
// The IQ3_S codebook as the kernels take it: 512 words, byte j of a word = magnitude j of the entry (1, 3, ..., 15).
void arcz_iq3s_grid(uint32_t* out) {
  for (int i = 0; i < 512; ++i)
    out[i] = (uint32_t)kIq3s.m[i][0] | ((uint32_t)kIq3s.m[i][1] << 8) | ((uint32_t)kIq3s.m[i][2] << 16) | ((uint32_t)kIq3s.m[i][3] << 24);
}

// The IQ3_XXS codebook as the kernels take it: 256 words, byte j of a word = magnitude j of the entry.
void arcz_iq3xxs_grid(uint32_t* out) {
  for (int i = 0; i < 256; ++i)
    out[i] = (uint32_t)kIq3xxs.m[i][0] | ((uint32_t)kIq3xxs.m[i][1] << 8) | ((uint32_t)kIq3xxs.m[i][2] << 16) | ((uint32_t)kIq3xxs.m[i][3] << 24);
}

// GGUF rows -> device planes (layout: kernels/common.h).  0 or -1 (unsupported type / K).
int arcz_repack_planes(uint32_t type, size_t rows, int K, const uint8_t* src, uint8_t* dst) {
  if (K <= 0 || K % 256) return -1;
  const int nsb = K / 256;
  const int64_t u = (int64_t)rows * nsb;
  if (type == QT_Q4_K || type == QT_Q5_K) {
    const PlanesQ4K pl = planes_q4k(rows, nsb);
    const bool q5 = type == QT_Q5_K;
    const size_t sbb = q5 ? 176 : 144;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i) {
      // header: d, dmin, then the 6-bit scales and mins (GGUF packing, reference src/quants.h:61-69) regrouped as
      // eight 12-bit entries sc | mn << 6
      const uint8_t* q = src + i * sbb + 4;
      uint8_t* h = dst + pl.hdr + i * 16;
      memcpy(h, src + i * sbb, 4);
      uint32_t w[3] = {0, 0, 0};
      for (int b = 0; b < 8; ++b) {
        const uint32_t sc = b < 4 ? (q[b] & 63u) : ((q[b + 4] & 0xFu) | ((uint32_t)(q[b - 4] >> 6) << 4));
        const uint32_t mn = b < 4 ? (q[b + 4] & 63u) : ((uint32_t)(q[b + 4] >> 4) | ((uint32_t)(q[b] >> 6) << 4));
        const uint64_t e = (uint64_t)(sc | (mn << 6)) << ((12 * b) & 31);
        w[(12 * b) >> 5] |= (uint32_t)e;
        if (((12 * b) >> 5) < 2) w[((12 * b) >> 5) + 1] |= (uint32_t)(e >> 32);
      }
      memcpy(h + 4, w, 12);
      memcpy(dst + pl.qs + i * 128, src + i * sbb + (q5 ? 48 : 16), 128);
      if (q5) {
        // fifth bits (reference src/quants.h:101-108: bit b of byte l of qh = element 32 b + l) regrouped per 16-byte
        // unit of nibbles: unit 2 j + half holds bytes l = 16 half .. 16 half + 15 of chunk j, low nibbles = block 2 j,
        // high nibbles = block 2 j + 1; byte m = 4 k + c of the unit gives bits 4 + k and k of byte c of the word
        const uint8_t* qh = src + i * sbb + 16;
        uint32_t H[8];
        for (int un = 0; un < 8; ++un) {
          const int j = un >> 1, half = un & 1;
          uint32_t word = 0;
          for (int m = 0; m < 16; ++m) {
            const int l = 16 * half + m, k = m >> 2, c = m & 3;
            word |= (uint32_t)((qh[l] >> (2 * j)) & 1) << (8 * c + 4 + k);
            word |= (uint32_t)((qh[l] >> (2 * j + 1)) & 1) << (8 * c + k);
          }
          H[un] = word;
        }
        memcpy(dst + pl.qh + i * 32, H, 32);
      }
    }
    return 0;
  }
  if (type == GGML_TYPE_IQ3_XXS) {
    // 98 bytes per superblock (f16 d, 64 index bytes, 8 words of sign codes and scales; reference
    // src/quants.h:220-239) -> the three fields as planes
    const PlanesIQ3XXS pl = planes_iq3xxs(rows, nsb);
    memset(dst + pl.d + u * 2, 0, raw_planes_bytes(QT_IQ3_XXS, rows, nsb) - (pl.d + u * 2));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i) {
      const uint8_t* p = src + i * 98;
      memcpy(dst + pl.d + i * 2, p, 2);
      memcpy(dst + pl.qs + i * 64, p + 2, 64);
      memcpy(dst + pl.ss + i * 32, p + 66, 32);
    }
    return 0;
  }
  if (type == GGML_TYPE_Q3_K) {
    // 110 bytes per superblock (hmask[32]: bit b of byte e = the third bit of element e of block b; qs[64]: byte
    // 32 (b / 4) + e, bits 2 (b % 4): its low two; sixteen 6-bit scales in 12 bytes; f16 d -- reference
    // src/quants.h:465-494) -> a block's bits together: two words of bit pairs, a word of third bits, a 12-bit entry of
    // its two scales (layout: kernels/common.h)
    const PlanesIQ3S pl = planes_iq3s(rows, nsb);
    memset(dst + pl.d + u * 2, 0, raw_planes_bytes(QT_Q3_K, rows, nsb) - (pl.d + u * 2));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i) {
      const uint8_t *p = src + i * 110, *hm = p, *qs = p + 32, *sc = p + 96;
      for (int b = 0; b < 8; ++b) {
        uint32_t D[2] = {0, 0}, H = 0;
        for (int j = 0; j < 32; ++j) {
          const uint32_t q2 = (qs[32 * (b / 4) + j] >> (2 * (b % 4))) & 3u, hb = (hm[j] >> b) & 1u;
          D[j >> 4] |= q2 << (8 * (j & 3) + 2 * ((j & 15) >> 2));
          H |= hb << (8 * (j & 3) + (j >> 2));
        }
        memcpy(dst + pl.qs + i * 64 + b * 8, D, 8);
        memcpy(dst + pl.sg + i * 32 + b * 4, &H, 4);
      }
      uint8_t hd[12] = {0};
      for (int k = 0; k < 16; ++k) {  // scale k: 6 bits at bit 6 k of the 96
        const uint32_t s6 = ((sc[k & 7] >> (4 * (k >> 3))) & 0xFu) | (((sc[8 + (k & 3)] >> (2 * (k >> 2))) & 3u) << 4);
        const int bit = 6 * k;
        hd[bit >> 3] |= (uint8_t)(s6 << (bit & 7));
        if ((bit & 7) > 2) hd[(bit >> 3) + 1] |= (uint8_t)(s6 >> (8 - (bit & 7)));
      }
      memcpy(dst + pl.hd + i * 12, hd, 12);
      memcpy(dst + pl.d + i * 2, p + 108, 2);
    }
    return 0;
  }
  if (type == QT_Q6_K) {
    const PlanesQ6K pl = planes_q6k(rows, nsb);
    memset(dst + pl.d + u * 2, 0, raw_planes_bytes(QT_Q6_K, rows, nsb) - (pl.d + u * 2));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i) {
      memcpy(dst + pl.ql + i * 128, src + i * 210, 128);
      memcpy(dst + pl.qh + i * 64, src + i * 210 + 128, 64);
      memcpy(dst + pl.sc + i * 16, src + i * 210 + 192, 16);
      memcpy(dst + pl.d + i * 2, src + i * 210 + 208, 2);
    }
    return 0;
  }
  if (type == GGML_TYPE_IQ3_S) {
    // 110-byte superblocks (f16 d, 64 index bytes, 8 bytes of ninth bits, 32 sign bytes, 4 bytes of scale nibbles;
    // reference src/quants.h:240-262) regrouped into planes, byte for byte
    const PlanesIQ3S pl = planes_iq3s(rows, nsb);
    memset(dst + pl.d + u * 2, 0, raw_planes_bytes(QT_IQ3_S, rows, nsb) - (pl.d + u * 2));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i) {
      const uint8_t* p = src + i * 110;
      memcpy(dst + pl.d + i * 2, p, 2);
      memcpy(dst + pl.qs + i * 64, p + 2, 64);
      memcpy(dst + pl.hd + i * 12, p + 66, 8);
      memcpy(dst + pl.sg + i * 32, p + 74, 32);
      memcpy(dst + pl.hd + i * 12 + 8, p + 106, 4);
    }
    return 0;
  }
  if (type == QT_IQ4_XS) {
    const PlanesIQ4XS pl = planes_iq4xs(rows, nsb);
    memset(dst + pl.hdr + u * 8, 0, raw_planes_bytes(QT_IQ4_XS, rows, nsb) - (pl.hdr + u * 8));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i) {
      memcpy(dst + pl.hdr + i * 8, src + i * 136, 8);
      memcpy(dst + pl.qs + i * 128, src + i * 136 + 8, 128);
    }
    return 0;
  }
  if (type == QT_Q8_0) {
    const PlanesQ80 pl = planes_q80(rows, nsb);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i)
      for (int b = 0; b < 8; ++b) {
        memcpy(dst + pl.d + i * 16 + 2 * b, src + i * 272 + 34 * b, 2);
        memcpy(dst + pl.qs + i * 256 + 32 * b, src + i * 272 + 34 * b + 2, 32);
      }
    return 0;
  }
  if (type == GGML_TYPE_MXFP4) {
    // eight 17-byte blocks (E8M0 scale byte, 16 bytes of nibbles: low = elements 0..15, high = 16..31, each an E2M1
    // code; reference src/quants.h:520-530) -> 128 bytes of nibbles and 8 scale bytes per superblock
    const PlanesMXFP4 pl = planes_mxfp4(rows, nsb);
    memset(dst + pl.e + u * 8, 0, raw_planes_bytes(QT_MXFP4, rows, nsb) - (pl.e + u * 8));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i)
      for (int b = 0; b < 8; ++b) {
        const uint8_t* blk = src + i * 136 + 17 * b;
        dst[pl.e + i * 8 + b] = blk[0];
        memcpy(dst + pl.qs + i * 128 + 16 * b, blk + 1, 16);
      }
    return 0;
  }
  if (type == GGML_TYPE_Q4_0 || type == GGML_TYPE_IQ4_NL) {
    // eight 18-byte blocks (f16 d, 16 bytes of nibbles: low = elements 0..15, high = 16..31; Q4_0: value = nibble - 8,
    // IQ4_NL: the nibble's entry of the IQ4 table; reference src/quants.h:136-148, 594-606) -> 128 bytes of nibbles and
    // 8 scales per superblock
    const PlanesQ40 pl = planes_q40(rows, nsb);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < u; ++i)
      for (int b = 0; b < 8; ++b) {
        const uint8_t* blk = src + i * 144 + 18 * b;
        memcpy(dst + pl.d + i * 16 + 2 * b, blk, 2);
        memcpy(dst + pl.qs + i * 128 + 16 * b, blk + 2, 16);
      }
    return 0;
  }
  return -1;
}

// Two types that share Q4_0's arithmetic -- one f16 scale times a small integer -- written out as Q4_0 blocks, value
// for value: AR4_128 (blocks of 128: f16 d, then four runs of 16 nibble bytes arranged as Q4_0's, value d * (q - 8);
// reference src/quants.h:531-542) gives each of its four runs the block's d; Q2_0 (blocks of 64: f16 d, 64 2-bit codes,
// element j in bits 2 (j % 4) of byte j / 4, value d * (q - 1); src/quants.h:607-616) becomes two blocks of nibbles
// q + 7.  K in whole source blocks; dst holds rows * K / 32 blocks of 18 bytes.  Bytes per 256 values: 132 and 72
// in the file, 144 as written here.  Returns the bytes of the source it read, 0 for another type or a K that does not fit.
size_t arcz_relayout_q4_0(uint32_t type, size_t rows, int K, const uint8_t* src, uint8_t* dst) {
  if (K <= 0) return 0;
  if (type == GGML_TYPE_AR4_128) {
    if (K % 128) return 0;
    const int64_t nb = (int64_t)rows * (K / 128);
    if (!dst) return (size_t)nb * 66;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nb; ++i) {
      const uint8_t* b = src + i * 66;
      for (int c = 0; c < 4; ++c) {
        uint8_t* o = dst + (i * 4 + c) * 18;
        memcpy(o, b, 2);
        memcpy(o + 2, b + 2 + 16 * c, 16);
      }
    }
    return (size_t)nb * 66;
  }
  if (type == GGML_TYPE_Q2_0) {
    if (K % 64) return 0;
    const int64_t nb = (int64_t)rows * (K / 64);
    if (!dst) return (size_t)nb * 18;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nb; ++i) {
      const uint8_t* b = src + i * 18;
      for (int c = 0; c < 2; ++c) {
        uint8_t* o = dst + (i * 2 + c) * 18;
        memcpy(o, b, 2);
        for (int j = 0; j < 16; ++j) {
          const int e0 = 32 * c + j, e1 = e0 + 16;
          const int q0 = (b[2 + e0 / 4] >> (2 * (e0 % 4))) & 3, q1 = (b[2 + e1 / 4] >> (2 * (e1 % 4))) & 3;
          o[2 + j] = (uint8_t)((q0 + 7) | ((q1 + 7) << 4));
        }
      }
    }
    return (size_t)nb * 18;
  }
  return 0;
}

// n values ~ N(mean, std): SplitMix64 -> two uniforms -> Box-Muller in f32, element i from the stream position i / 2
// (so any sub-range can be generated alone).  The same seed gives the same tensor on every machine.
void arcz_gen_normal(uint64_t seed, size_t n, float mean, float std, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < (int64_t)((n + 1) / 2); ++p) {
    uint64_t s = seed * 0xD1342543DE82EF95ull + (uint64_t)p * 0x9E3779B97F4A7C15ull * 2;
    const uint64_t a = splitmix64(s), b = splitmix64(s);
    const float u1 = ((float)((a >> 40) + 1)) * (1.0f / 16777216.0f);  // (0, 1]
    const float u2 = (float)(b >> 40) * (1.0f / 16777216.0f);          // [0, 1)
    const float r = sqrtf(-2.0f * logf(u1)), th = 6.28318530717958647692f * u2;
    out[2 * p] = mean + std * r * cosf(th);
    if ((size_t)(2 * p + 1) < n) out[2 * p + 1] = mean + std * r * sinf(th);
  }
}

// f32 rows [N][K] -> GGUF Q8_0 (34-byte blocks): d = amax / 127 kept as fp16, q = rte(v * (1 / d)) with the f32 d
// (reference src/quants.h:429-442).
void arcz_quantize_q8_0(const float* src, size_t N, int K, uint8_t* out) {
  const int64_t nb = (int64_t)N * (K / 32);
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < nb; ++b) {
    const float* v = src + b * 32;
    float amax = 0;
    for (int i = 0; i < 32; ++i) amax = std::fmax(amax, std::fabs(v[i]));
    const float d = amax / 127.0f, inv = d > 0 ? 1.0f / d : 0.0f;
    uint8_t* blk = out + b * 34;
    const uint16_t dh = f32_to_f16(d);
    memcpy(blk, &dh, 2);
    for (int i = 0; i < 32; ++i) blk[2 + i] = (uint8_t)(int8_t)std::lrintf(v[i] * inv);
  }
}

// f32 rows -> GGUF Q4_K superblocks (144 bytes per 256 values).  Per 32-block: offset lo = min(v, 0), step
// (max - lo) / 15; the eight steps and offsets are rounded to 6 bits against d = max step / 63, dmin = max offset / 63
// (both kept as fp16); quants re-rounded against the stored scales.  Layout as GGUF (reference src/quants.h:61-69,
// 91-113).
void arcz_quantize_q4_k(const float* src, size_t N, int K, uint8_t* out) {
  const int64_t nsbt = (int64_t)N * (K / 256);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < nsbt; ++s) {
    const float* v = src + s * 256;
    uint8_t* p = out + s * 144;
    float step[8], off[8], smax = 0, omax = 0;
    for (int b = 0; b < 8; ++b) {
      float lo = 0, hi = 0;
      for (int i = 0; i < 32; ++i) { lo = std::fmin(lo, v[32 * b + i]); hi = std::fmax(hi, v[32 * b + i]); }
      step[b] = (hi - lo) / 15.0f;
      off[b] = -lo;
      smax = std::fmax(smax, step[b]);
      omax = std::fmax(omax, off[b]);
    }
    const uint16_t dh = f32_to_f16(smax / 63.0f), mh = f32_to_f16(omax / 63.0f);
    const float d = f16_to_f32(dh), dmin = f16_to_f32(mh);
    int sc[8], mn[8];
    for (int b = 0; b < 8; ++b) {
      sc[b] = d > 0 ? std::min(63, std::max(0, (int)std::lrintf(step[b] / d))) : 0;
      mn[b] = dmin > 0 ? std::min(63, std::max(0, (int)std::lrintf(off[b] / dmin))) : 0;
    }
    memcpy(p, &dh, 2);
    memcpy(p + 2, &mh, 2);
    uint8_t* q = p + 4;
    memset(q, 0, 12);
    for (int j = 0; j < 8; ++j) {
      if (j < 4) {
        q[j] |= sc[j] & 63;
        q[j + 4] |= mn[j] & 63;
      } else {
        q[j + 4] = (uint8_t)((sc[j] & 0xF) | ((mn[j] & 0xF) << 4));
        q[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
        q[j] |= (uint8_t)((mn[j] >> 4) << 6);
      }
    }
    uint8_t* qs = p + 16;
    for (int j = 0; j < 4; ++j)
      for (int l = 0; l < 32; ++l) {
        int qq[2];
        for (int h = 0; h < 2; ++h) {
          const int b = 2 * j + h;
          const float sd = d * (float)sc[b], x = v[64 * j + 32 * h + l] + dmin * (float)mn[b];
          qq[h] = sd > 0 ? std::min(15, std::max(0, (int)std::lrintf(x / sd))) : 0;
        }
        qs[32 * j + l] = (uint8_t)(qq[0] | (qq[1] << 4));
      }
  }
}

// f32 rows -> GGUF Q5_K superblocks (176 bytes per 256 values): as Q4_K with 31 steps per block; the fifth bit of
// element 32 b + l is bit b of byte l of the 32 bytes between the scales and the nibbles (reference
// src/quants.h:101-108).
void arcz_quantize_q5_k(const float* src, size_t N, int K, uint8_t* out) {
  const int64_t nsbt = (int64_t)N * (K / 256);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < nsbt; ++s) {
    const float* v = src + s * 256;
    uint8_t* p = out + s * 176;
    float step[8], off[8], smax = 0, omax = 0;
    for (int b = 0; b < 8; ++b) {
      float lo = 0, hi = 0;
      for (int i = 0; i < 32; ++i) { lo = std::fmin(lo, v[32 * b + i]); hi = std::fmax(hi, v[32 * b + i]); }
      step[b] = (hi - lo) / 31.0f;
      off[b] = -lo;
      smax = std::fmax(smax, step[b]);
      omax = std::fmax(omax, off[b]);
    }
    const uint16_t dh = f32_to_f16(smax / 63.0f), mh = f32_to_f16(omax / 63.0f);
    const float d = f16_to_f32(dh), dmin = f16_to_f32(mh);
    int sc[8], mn[8];
    for (int b = 0; b < 8; ++b) {
      sc[b] = d > 0 ? std::min(63, std::max(0, (int)std::lrintf(step[b] / d))) : 0;
      mn[b] = dmin > 0 ? std::min(63, std::max(0, (int)std::lrintf(off[b] / dmin))) : 0;
    }
    memcpy(p, &dh, 2);
    memcpy(p + 2, &mh, 2);
    uint8_t* q = p + 4;
    memset(q, 0, 12 + 32);
    for (int j = 0; j < 8; ++j) {
      if (j < 4) {
        q[j] |= sc[j] & 63;
        q[j + 4] |= mn[j] & 63;
      } else {
        q[j + 4] = (uint8_t)((sc[j] & 0xF) | ((mn[j] & 0xF) << 4));
        q[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
        q[j] |= (uint8_t)((mn[j] >> 4) << 6);
      }
    }
    uint8_t *qh = p + 16, *qs = p + 48;
    for (int j = 0; j < 4; ++j)
      for (int l = 0; l < 32; ++l) {
        int qq[2];
        for (int h = 0; h < 2; ++h) {
          const int b = 2 * j + h;
          const float sd = d * (float)sc[b], x = v[64 * j + 32 * h + l] + dmin * (float)mn[b];
          qq[h] = sd > 0 ? std::min(31, std::max(0, (int)std::lrintf(x / sd))) : 0;
          qh[l] |= (uint8_t)((qq[h] >> 4) << b);
        }
        qs[32 * j + l] = (uint8_t)((qq[0] & 15) | ((qq[1] & 15) << 4));
      }
  }
}

// f32 rows -> GGUF Q6_K superblocks (210 bytes per 256 values): per 16 values a step amax / 31, rounded to int8
// against d = max step / 127 (fp16); q = rte(v / (d * sc)) in -32..31, stored + 32 (reference src/quants.h:115-134).
void arcz_quantize_q6_k(const float* src, size_t N, int K, uint8_t* out) {
  const int64_t nsbt = (int64_t)N * (K / 256);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < nsbt; ++s) {
    const float* v = src + s * 256;
    uint8_t* p = out + s * 210;
    float step[16], smax = 0;
    for (int b = 0; b < 16; ++b) {
      float amax = 0;
      for (int i = 0; i < 16; ++i) amax = std::fmax(amax, std::fabs(v[16 * b + i]));
      step[b] = amax / 31.0f;
      smax = std::fmax(smax, step[b]);
    }
    const uint16_t dh = f32_to_f16(smax / 127.0f);
    const float d = f16_to_f32(dh);
    int8_t sc[16];
    int q[256];
    for (int b = 0; b < 16; ++b) {
      sc[b] = (int8_t)(d > 0 ? std::min(127, std::max(1, (int)std::lrintf(step[b] / d))) : 0);
      const float sd = d * (float)sc[b];
      for (int i = 0; i < 16; ++i)
        q[16 * b + i] = 32 + (sd > 0 ? std::min(31, std::max(-32, (int)std::lrintf(v[16 * b + i] / sd))) : 0);
    }
    q6k_pack(q, p, p + 128);
    memcpy(p + 192, sc, 16);
    memcpy(p + 208, &dh, 2);
  }
}

// f32 rows -> GGUF IQ4_XS superblocks (136 bytes per 256 values; reference src/quants.h:297-311): per 32-block a step
// amax / 127 (the table's largest magnitude), rounded to 1..31 against d = max step / 31 (fp16) and stored + 32 in six
// bits (low four in one nibble, high two in the 16-bit word), each value as the code of the nearest table entry.
void arcz_quantize_iq4_xs(const float* src, size_t N, int K, uint8_t* out) {
  static const int kv[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
  const int64_t nsbt = (int64_t)N * (K / 256);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < nsbt; ++s) {
    const float* v = src + s * 256;
    uint8_t* p = out + s * 136;
    float step[8], smax = 0;
    for (int b = 0; b < 8; ++b) {
      float amax = 0;
      for (int i = 0; i < 32; ++i) amax = std::fmax(amax, std::fabs(v[32 * b + i]));
      step[b] = amax / 127.0f;
      smax = std::fmax(smax, step[b]);
    }
    const uint16_t dh = f32_to_f16(smax / 31.0f);
    const float d = f16_to_f32(dh);
    memset(p, 0, 136);
    memcpy(p, &dh, 2);
    uint16_t sh = 0;
    for (int b = 0; b < 8; ++b) {
      const int l = d > 0 ? std::min(31, std::max(1, (int)std::lrintf(step[b] / d))) : 0;
      const int ls = l + 32;
      p[4 + b / 2] |= (uint8_t)((ls & 0xF) << (4 * (b % 2)));
      sh |= (uint16_t)((ls >> 4) << (2 * b));
      const float sd = d * (float)l;
      for (int i = 0; i < 32; ++i) {
        int best = 8;
        if (sd > 0) {
          const float x = v[32 * b + i] / sd;
          float be = 1e30f;
          for (int c = 0; c < 16; ++c) {
            const float e = std::fabs(x - (float)kv[c]);
            if (e < be) { be = e; best = c; }
          }
        }
        p[8 + 16 * b + (i & 15)] |= (uint8_t)(best << (4 * (i >> 4)));
      }
    }
    memcpy(p + 2, &sh, 2);
  }
}

// f32 rows -> GGUF IQ3_S superblocks (110 bytes per 256 values; reference src/quants.h:240-262): per 32-block a step
// amax / 15 (the codebook's largest magnitude), d = max step / 31 (fp16), sub-scale 1 + 2 s with s = the nearest of
// 0..15; each 4 values take the codebook entry nearest to their magnitudes (all 512 tried), signs apart.  An input
// generator for tests: no search over scales as a real quantizer would make.
void arcz_quantize_iq3_s(const float* src, size_t N, int K, uint8_t* out) {
  const int64_t nsbt = (int64_t)N * (K / 256);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < nsbt; ++s) {
    const float* v = src + s * 256;
    uint8_t* p = out + s * 110;
    memset(p, 0, 110);
    float step[8], smax = 0;
    for (int b = 0; b < 8; ++b) {
      float amax = 0;
      for (int i = 0; i < 32; ++i) amax = std::fmax(amax, std::fabs(v[32 * b + i]));
      step[b] = amax / 15.0f;
      smax = std::fmax(smax, step[b]);
    }
    const uint16_t dh = f32_to_f16(smax / 31.0f);
    const float d = f16_to_f32(dh);
    memcpy(p, &dh, 2);
    for (int b = 0; b < 8; ++b) {
      const int sn = d > 0 ? std::min(15, std::max(0, (int)std::lrintf((step[b] / d - 1.0f) * 0.5f))) : 0;
      p[106 + b / 2] |= (uint8_t)(sn << (4 * (b % 2)));
      const float sd = d * (float)(1 + 2 * sn), inv = sd > 0 ? 1.0f / sd : 0.0f;
      for (int g = 0; g < 8; ++g) {
        float a[4];
        for (int j = 0; j < 4; ++j) {
          const float x = v[32 * b + 4 * g + j];
          a[j] = std::fabs(x) * inv;
          if (x < 0) p[74 + 4 * b + (4 * g + j) / 8] |= (uint8_t)(1u << ((4 * g + j) % 8));
        }
        int best = 0;
        float bd = 1e30f;
        for (int i = 0; i < 512; ++i) {
          float e = 0;
          for (int j = 0; j < 4; ++j) e += (a[j] - (float)kIq3s.m[i][j]) * (a[j] - (float)kIq3s.m[i][j]);
          if (e < bd) { bd = e; best = i; }
        }
        p[2 + 8 * b + g] = (uint8_t)(best & 255);
        p[66 + b] |= (uint8_t)((best >> 8) << g);
      }
    }
  }
}

// f32 rows -> GGUF Q4_0 blocks the way the reference makes them (src/quants.h:444-463, llama.cpp's
// quantize_row_q4_0_ref): d = (the value of largest magnitude) / -8, q = min(15, (int)(v / d + 8.5)).
static void arcz_quantize_q4_0(const float* src, size_t N, int K, uint8_t* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < (int64_t)(N * (size_t)(K / 32)); ++b) {
    const float* v = src + b * 32;
    float amax = 0.0f, mx = 0.0f;
    for (int i = 0; i < 32; ++i)
      if (std::fabs(v[i]) > amax) { amax = std::fabs(v[i]); mx = v[i]; }
    const float d = mx / -8.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t* blk = out + b * 18;
    const uint16_t dh = f32_to_f16(d);
    memcpy(blk, &dh, 2);
    for (int i = 0; i < 16; ++i) {
      const int q0 = std::min(15, (int)(v[i] * id + 8.5f)), q1 = std::min(15, (int)(v[i + 16] * id + 8.5f));
      blk[2 + i] = (uint8_t)(q0 | (q1 << 4));
    }
  }
}

// f32 rows -> GGUF IQ3_XXS superblocks (98 bytes per 256 values; reference src/quants.h:220-239): per 32-block a step
// amax / 62 (the codebook's largest magnitude), d / 4 = max step / 31 (d an fp16), the scale s the nearest of 0..15 to
// (step / (d / 4) - 1) / 2; each 4 values take the codebook entry nearest to their magnitudes (all 256 tried); of each 8
// values the signs as a 7-bit code whose parity is the eighth's -- where the eight signs are an odd number of minus
// signs, the value of smallest magnitude changes its sign.  An input generator for tests.
static void arcz_quantize_iq3_xxs(const float* src, size_t N, int K, uint8_t* out) {
  const int64_t nsbt = (int64_t)N * (K / 256);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < nsbt; ++s) {
    const float* v = src + s * 256;
    uint8_t* p = out + s * 98;
    memset(p, 0, 98);
    float step[8], smax = 0;
    for (int b = 0; b < 8; ++b) {
      float amax = 0;
      for (int i = 0; i < 32; ++i) amax = std::fmax(amax, std::fabs(v[32 * b + i]));
      step[b] = amax / 62.0f;
      smax = std::fmax(smax, step[b]);
    }
    const uint16_t dh = f32_to_f16(4.0f * smax / 31.0f);
    const float d4 = f16_to_f32(dh) / 4.0f;
    memcpy(p, &dh, 2);
    for (int b = 0; b < 8; ++b) {
      const int sn = d4 > 0 ? std::min(15, std::max(0, (int)std::lrintf((step[b] / d4 - 1.0f) * 0.5f))) : 0;
      const float sd = d4 * (float)(1 + 2 * sn), inv = sd > 0 ? 1.0f / sd : 0.0f;
      uint32_t a = (uint32_t)sn << 28;
      for (int l = 0; l < 4; ++l) {
        uint32_t sg = 0;
        int least = 0;
        for (int j = 0; j < 8; ++j) {
          const float x = v[32 * b + 8 * l + j];
          if (x < 0) sg |= 1u << j;
          if (std::fabs(x) < std::fabs(v[32 * b + 8 * l + least])) least = j;
        }
        if (__builtin_popcount(sg) & 1) sg ^= 1u << least;
        a |= (sg & 127u) << (7 * l);
        for (int h = 0; h < 2; ++h) {
          float m[4];
          for (int j = 0; j < 4; ++j) m[j] = std::fabs(v[32 * b + 8 * l + 4 * h + j]) * inv;
          int best = 0;
          float bd = 1e30f;
          for (int i = 0; i < 256; ++i) {
            float e = 0;
            for (int j = 0; j < 4; ++j) e += (m[j] - (float)kIq3xxs.m[i][j]) * (m[j] - (float)kIq3xxs.m[i][j]);
            if (e < bd) { bd = e; best = i; }
          }
          p[2 + 8 * b + 2 * l + h] = (uint8_t)best;
        }
      }
      memcpy(p + 66 + 4 * b, &a, 4);
    }
  }
}

// f32 rows -> GGUF Q3_K superblocks (110 bytes per 256 values; reference src/quants.h:465-494): per 16 values a step
// (the value of largest magnitude) / -4, which that value then decodes to exactly; d = the largest |step| / 31 (fp16),
// the 6-bit scale round(step / d) + 32; each value the nearest of -4..3 steps.  An input generator for tests.
static void arcz_quantize_q3_k(const float* src, size_t N, int K, uint8_t* out) {
  const int64_t nsbt = (int64_t)N * (K / 256);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < nsbt; ++s) {
    const float* v = src + s * 256;
    uint8_t* p = out + s * 110;
    memset(p, 0, 110);
    float step[16], smax = 0;
    for (int b = 0; b < 16; ++b) {
      float amax = 0, mx = 0;
      for (int i = 0; i < 16; ++i)
        if (std::fabs(v[16 * b + i]) > amax) { amax = std::fabs(v[16 * b + i]); mx = v[16 * b + i]; }
      step[b] = mx / -4.0f;
      smax = std::fmax(smax, std::fabs(step[b]));
    }
    const uint16_t dh = f32_to_f16(smax / 31.0f);
    const float d = f16_to_f32(dh);
    memcpy(p + 108, &dh, 2);
    for (int b = 0; b < 16; ++b) {
      const int sc = d > 0 ? std::min(31, std::max(-32, (int)std::lrintf(step[b] / d))) : 0, s6 = sc + 32;
      p[96 + (b & 7)] |= (uint8_t)((s6 & 0xF) << (4 * (b >> 3)));
      p[104 + (b & 3)] |= (uint8_t)((s6 >> 4) << (2 * (b >> 2)));
      const float sd = d * (float)sc, inv = sd != 0 ? 1.0f / sd : 0.0f;
      for (int i = 0; i < 16; ++i) {
        const int e = 16 * b + i, blk = e >> 5, el = e & 31;
        const int q = std::min(3, std::max(-4, (int)std::lrintf(v[e] * inv))) + 4;  // 0..7
        p[32 + 32 * (blk / 4) + el] |= (uint8_t)((q & 3) << (2 * (blk % 4)));
        if (q & 4) p[el] |= (uint8_t)(1u << blk);
      }
    }
  }
}

// f32 rows -> GGUF IQ4_NL blocks (18 bytes per 32 values; reference src/quants.h:594-606): d = (the value of largest
// magnitude) / -127, which that value then decodes to exactly; every value takes the nearest entry of the table.  An
// input generator for tests: no search over scales as a real quantizer would make.
static void arcz_quantize_iq4_nl(const float* src, size_t N, int K, uint8_t* out) {
  static const int kv[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < (int64_t)(N * (size_t)(K / 32)); ++b) {
    const float* v = src + b * 32;
    float amax = 0.0f, mx = 0.0f;
    for (int i = 0; i < 32; ++i)
      if (std::fabs(v[i]) > amax) { amax = std::fabs(v[i]); mx = v[i]; }
    uint8_t* blk = out + b * 18;
    const uint16_t dh = f32_to_f16(mx / -127.0f);
    const float d = f16_to_f32(dh), id = d != 0.0f ? 1.0f / d : 0.0f;
    memcpy(blk, &dh, 2);
    memset(blk + 2, 0, 16);
    for (int i = 0; i < 32; ++i) {
      const float x = v[i] * id;
      int best = 0;
      float be = 1e30f;
      for (int c = 0; c < 16; ++c) {
        const float e = std::fabs(x - (float)kv[c]);
        if (e < be) { be = e; best = c; }
      }
      blk[2 + (i & 15)] |= (uint8_t)(best << (4 * (i >> 4)));
    }
  }
}

// f32 rows -> GGUF MXFP4 blocks (17 bytes per 32 values; reference src/quants.h:495-503, 520-530): the scale byte e is
// the smallest with amax <= 12 * 2^(e - 128) (12 = the table's largest entry), every value takes the nearest of
// +-{0, 1, 2, 3, 4, 6, 8, 12} * 2^(e - 128).  An input generator for tests.
static void arcz_quantize_mxfp4(const float* src, size_t N, int K, uint8_t* out) {
  static const int kv[8] = {0, 1, 2, 3, 4, 6, 8, 12};
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < (int64_t)(N * (size_t)(K / 32)); ++b) {
    const float* v = src + b * 32;
    float amax = 0.0f;
    for (int i = 0; i < 32; ++i) amax = std::fmax(amax, std::fabs(v[i]));
    int e = 0;
    if (amax > 0.0f) {
      int ex;
      const float m = std::frexp(amax / 12.0f, &ex);  // amax / 12 = m 2^ex, 0.5 <= m < 1
      e = std::min(254, std::max(0, (m == 0.5f ? ex - 1 : ex) + 128));
    }
    uint8_t* blk = out + b * 17;
    blk[0] = (uint8_t)e;
    memset(blk + 1, 0, 16);
    const float id = std::ldexp(1.0f, 128 - e);
    for (int i = 0; i < 32; ++i) {
      const float x = std::fabs(v[i]) * id;
      int best = 0;
      float be = 1e30f;
      for (int c = 0; c < 8; ++c) {
        const float er = std::fabs(x - (float)kv[c]);
        if (er < be) { be = er; best = c; }
      }
      if (v[i] < 0.0f && best) best |= 8;
      blk[1 + (i & 15)] |= (uint8_t)(best << (4 * (i >> 4)));
    }
  }
}

// Quantizes f32 rows to `type` (2, 8, 11, 12, 13, 14, 18, 20, 21, 23, 39).  0 or -1.
int arcz_quantize_rows(uint32_t type, const float* src, size_t N, int K, uint8_t* out) {
  if (K <= 0 || K % 256) return -1;
  if (type == GGML_TYPE_Q4_0) arcz_quantize_q4_0(src, N, K, out);
  else if (type == QT_Q8_0) arcz_quantize_q8_0(src, N, K, out);
  else if (type == QT_Q4_K) arcz_quantize_q4_k(src, N, K, out);
  else if (type == QT_Q5_K) arcz_quantize_q5_k(src, N, K, out);
  else if (type == QT_Q6_K) arcz_quantize_q6_k(src, N, K, out);
  else if (type == QT_IQ4_XS) arcz_quantize_iq4_xs(src, N, K, out);
  else if (type == GGML_TYPE_IQ3_S) arcz_quantize_iq3_s(src, N, K, out);
  else if (type == GGML_TYPE_Q3_K) arcz_quantize_q3_k(src, N, K, out);
  else if (type == GGML_TYPE_IQ3_XXS) arcz_quantize_iq3_xxs(src, N, K, out);
  else if (type == GGML_TYPE_IQ4_NL) arcz_quantize_iq4_nl(src, N, K, out);
  else if (type == GGML_TYPE_MXFP4) arcz_quantize_mxfp4(src, N, K, out);
  else return -1;
  return 0;
}

// Synthetic weights: rows [row0, row0 + N) of a matrix ~ N(0, std) with the given seed, quantized to `type`, written
// as GGUF blocks.  Generated in slabs so that a 150k-row matrix needs no f32 copy of itself.
int arcz_gen_weights(uint32_t type, uint64_t seed, size_t N, int K, float std, uint8_t* out) {
  if (K <= 0 || K % 256 || !arcz_gguf_bytes(type, 1, K)) return -1;
  const size_t slab = 4096, rb = arcz_gguf_bytes(type, 1, K);
  std::vector<float> f(slab * (size_t)K);
  for (size_t r0 = 0; r0 < N; r0 += slab) {
    const size_t nr = std::min(slab, N - r0);
    arcz_gen_normal(seed + 0x1000003ull * (r0 / slab + 1), nr * K, 0.0f, std, f.data());
    arcz_quantize_rows(type, f.data(), nr, K, out + r0 * rb);
  }
  return 0;
}

}  // extern "C"
