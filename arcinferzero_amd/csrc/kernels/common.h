// Shared device helpers for the gfx950 kernels: vector types, GGUF type ids, the device weight layout, scale decoding.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __HIPCC__
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
#endif

// GGUF type ids (reference src/gguf.h:18-22)
#define QT_Q4_0 2
#define QT_Q8_0 8
#define QT_Q3_K 11
#define QT_Q4_K 12
#define QT_Q5_K 13
#define QT_Q6_K 14
#define QT_IQ3_XXS 18
#define QT_IQ4_NL 20
#define QT_IQ3_S 21
#define QT_IQ4_XS 23
#define QT_MXFP4 39

// ---- device weight layout ("raw planes").  A matrix of R rows x K columns (K % 256 == 0, nsb = K / 256) is held
// as separate planes, each row-major over (row, superblock), so that every field is 16-byte aligned and a wave's
// consecutive lanes read consecutive 16-byte units.  The byte count equals the GGUF byte count except Q6_K's 2-byte
// scale per superblock, which keeps its size (the plane as a whole is padded to 16 bytes).
//   Q4_K : qs  [R][nsb][128]  (GGUF order: byte l of chunk j = element 64j+l low nibble, 64j+32+l high nibble)
//          hdr [R][nsb][16]   (f16 d, f16 dmin, then eight 12-bit entries sc_b | mn_b << 6 at bit 12 b: the 6-bit scale
//                              and min of sub-block b, regrouped from GGUF's packing so that the pair of entries of a
//                              64-element chunk is one 24-bit field)
//   Q5_K : qs and hdr as Q4_K (the low four bits of each value), then
//          qh  [R][nsb][8] words: word i holds the fifth bits of the 32 values of 16-byte unit i of qs, regrouped from
//                              GGUF's 32 bytes (bit b of byte l = element 32 b + l) so that a shift and one mask put
//                              them in place: byte c of the word, bit 4 + k = the low-nibble value of the unit's byte
//                              4 k + c, bit k = the high-nibble value of that byte (k = 0..3)
//   Q6_K : ql  [R][nsb][128], qh [R][nsb][64], sc [R][nsb][16] (int8), d [R][nsb] (f16)
//   Q8_0 : qs  [R][nsb][256] (int8), d [R][nsb][8] (f16)
//   IQ4_XS: qs [R][nsb][128]  (GGUF order: byte j of block b = element 32b+j low nibble, 32b+16+j high nibble; a nibble
//                              is a code of the 16-entry table below), hdr [R][nsb][8] (f16 d, 16 bits of the eight
//                              6-bit block scales' high parts, 4 bytes of their low nibbles: as GGUF)
//   Q4_0 : qs  [R][nsb][128]  (the sixteen nibble bytes of each of the superblock's eight 32-value blocks, as GGUF: byte
//                              j of block b = element 32b+j low nibble, 32b+16+j high nibble; value = nibble - 8),
//          d   [R][nsb][8] (f16: the eight blocks' scales).  144 bytes per 256 values, as GGUF's eight 18-byte blocks.
//   IQ3_XXS: qs [R][nsb][64]  (eight codebook indices per 32-value block, a byte each, each naming 4 magnitudes of
//                              4, 12, ..., 52, 62), ss [R][nsb][8] words (block b: four 7-bit sign codes -- the signs of 8
//                              values, the eighth making their number even -- and in the top nibble the scale s),
//          d   [R][nsb]       (f16).  value = d / 4 * (1 + 2 s) * the signed magnitude.  98 bytes per 256 values, as
//          GGUF (src/quants.h:220-239).
//   Q3_K : the planes of IQ3_S in size and place (planes_iq3s), regrouped from GGUF's hmask / qs / scales so that a
//          32-value block's bits lie together and four values come out of a word with a shift and a mask:
//          qs  [R][nsb][64]   (block b: words D0, D1 at bytes 8 b: value j of the block's first / second 16 in byte
//                              j % 4, bits 2 (j / 4) and the next: its low two bits),
//          sg  [R][nsb][32]   (block b: the word of third bits, value j (0..31) at bit 8 (j % 4) + j / 4),
//          hd  [R][nsb][12]   (eight 12-bit entries, entry b at bit 12 b: the 6-bit scales of the block's first and
//                              second 16 values, s | s' << 6, 32 not yet subtracted),
//          d   [R][nsb]       (f16).  110 bytes per 256 values, as GGUF (src/quants.h:465-494).
//          value = d * (scale - 32) * (the three bits - 4).
//   IQ4_NL: as Q4_0; value = the nibble's entry of the IQ4_XS table.
//   MXFP4: qs  [R][nsb][128]  (as Q4_0; a nibble is an E2M1 code: sign | 3 bits naming 0, 1, 2, 3, 4, 6, 8, 12, the
//                              doubled magnitudes), e [R][nsb][8] (the eight blocks' E8M0 scale bytes: value =
//                              2^(e - 128) * the table's entry).  136 bytes per 256 values, as GGUF's eight 17-byte blocks.
//   IQ3_S: qs  [R][nsb][64]   (the low bytes of the 64 codebook indices: 8 per 32-value block, each naming 4 magnitudes),
//          sg  [R][nsb][32]   (sign bits: 4 bytes per block, bit e of the block's 32 = element e is negative),
//          hd  [R][nsb][12]   (8 bytes of ninth index bits, bit g of byte b = index g of block b; 4 bytes of scale nibbles,
//                              nibble b = s of block b, sub-scale 1 + 2 s),
//          d   [R][nsb]       (f16).  110 bytes per 256 values, as GGUF (src/quants.h:240-262).
// Plane offsets from the start of the buffer, in bytes (each a multiple of 256 when R * nsb is a multiple of 16;
// always a multiple of 16 otherwise except as noted).
struct PlanesQ4K { size_t qs, hdr, qh; };  // (qh: Q5_K only)
struct PlanesQ6K { size_t ql, qh, sc, d; };
struct PlanesQ80 { size_t qs, d; };
struct PlanesIQ4XS { size_t qs, hdr; };
struct PlanesQ40 { size_t qs, d; };
struct PlanesIQ3S { size_t qs, sg, hd, d; };
struct PlanesMXFP4 { size_t qs, e; };
struct PlanesIQ3XXS { size_t qs, ss, d; };

__host__ __device__ inline size_t align16(size_t x) { return (x + 15) & ~(size_t)15; }
__host__ __device__ inline PlanesQ4K planes_q4k(size_t rows, int nsb) {
  PlanesQ4K p;
  p.qs = 0;
  p.hdr = rows * (size_t)nsb * 128;
  p.qh = rows * (size_t)nsb * 144;
  return p;
}
__host__ __device__ inline PlanesQ6K planes_q6k(size_t rows, int nsb) {
  PlanesQ6K p;
  const size_t u = rows * (size_t)nsb;
  p.ql = 0;
  p.qh = u * 128;
  p.sc = p.qh + u * 64;
  p.d = p.sc + u * 16;
  return p;
}
__host__ __device__ inline PlanesQ80 planes_q80(size_t rows, int nsb) {
  PlanesQ80 p;
  p.qs = 0;
  p.d = rows * (size_t)nsb * 256;
  return p;
}
__host__ __device__ inline PlanesIQ4XS planes_iq4xs(size_t rows, int nsb) {
  PlanesIQ4XS p;
  p.qs = 0;
  p.hdr = rows * (size_t)nsb * 128;
  return p;
}
__host__ __device__ inline PlanesQ40 planes_q40(size_t rows, int nsb) {
  PlanesQ40 p;
  p.qs = 0;
  p.d = rows * (size_t)nsb * 128;
  return p;
}
__host__ __device__ inline PlanesMXFP4 planes_mxfp4(size_t rows, int nsb) {
  PlanesMXFP4 p;
  p.qs = 0;
  p.e = rows * (size_t)nsb * 128;
  return p;
}
__host__ __device__ inline PlanesIQ3XXS planes_iq3xxs(size_t rows, int nsb) {
  PlanesIQ3XXS p;
  const size_t u = rows * (size_t)nsb;
  p.qs = 0;
  p.ss = u * 64;
  p.d = u * 96;
  return p;
}
__host__ __device__ inline PlanesIQ3S planes_iq3s(size_t rows, int nsb) {
  PlanesIQ3S p;
  const size_t u = rows * (size_t)nsb;
  p.qs = 0;
  p.sg = u * 64;
  p.hd = u * 96;
  p.d = u * 108;
  return p;
}
__host__ __device__ inline size_t raw_planes_bytes(int qt, size_t rows, int nsb) {
  const size_t u = rows * (size_t)nsb;
  if (qt == QT_IQ3_S || qt == QT_Q3_K) return align16(u * 110);
  if (qt == QT_IQ3_XXS) return align16(u * 98);
  if (qt == QT_Q4_0 || qt == QT_IQ4_NL) return u * 144;
  if (qt == QT_MXFP4) return align16(u * 136);
  if (qt == QT_Q4_K) return u * 144;
  if (qt == QT_Q5_K) return u * 176;
  if (qt == QT_Q6_K) return align16(u * 208 + u * 2);
  if (qt == QT_Q8_0) return u * 272;
  if (qt == QT_IQ4_XS) return align16(u * 136);
  return 0;
}

#ifdef __HIPCC__
__device__ inline float f16_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)(h & 0xFFFFu));
}

// Per-byte (q - 32) for four 6-bit unsigned values packed in a word, without borrows between bytes.
__device__ inline uint32_t sub32_bytes(uint32_t q) { return ((q | 0x80808080u) - 0x20202020u) ^ 0x80808080u; }

// 6-bit scale and min of Q4_K sub-blocks 2j and 2j+1 from the three words of entries of the device header
// (bits 24 j .. 24 j + 23 of the 96-bit string s0 | s1 << 32 | s2 << 64).  Branch-free: j differs between lanes.
__device__ inline void q4k_scales_pair(uint32_t s0, uint32_t s1, uint32_t s2, int j, int& sc0, int& sc1, int& mn0,
                                       int& mn1) {
  const uint32_t lo = j < 2 ? s0 : (j == 2 ? s1 : s2), hi = j < 2 ? s1 : s2;
  const uint32_t g = __builtin_amdgcn_alignbit(hi, lo, (24 * j) & 31);
  sc0 = g & 63;
  mn0 = (g >> 6) & 63;
  sc1 = (g >> 12) & 63;
  mn1 = (g >> 18) & 63;
}

// Q5_K: word k (0..3) of a 16-byte unit of nibbles with the fifth bits from the unit's word H of the qh plane: the 16
// values of the low nibbles, and of the high nibbles, as four bytes 0..31 each.
__device__ inline uint32_t q5k_lo(uint32_t w, uint32_t H, int k) { return (w & 0x0F0F0F0Fu) | ((H >> k) & 0x10101010u); }
__device__ inline uint32_t q5k_hi(uint32_t w, uint32_t H, int k) {
  return ((w >> 4) & 0x0F0F0F0Fu) | ((H << (4 - k)) & 0x10101010u);
}

// IQ4_XS: four 4-bit codes, one in the low nibble of each byte of c, to the four int8 values of the format's table
// (-127 -104 -83 -65 -49 -35 -22 -10 | 1 13 25 38 53 69 89 113; reference src/iq_tables.h:364-367): a byte permute per
// table half, the code's bit 3 picks between them.
__device__ inline uint32_t iq4_lookup(uint32_t c) {
  const uint32_t sel = c & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, sel);  // codes 0-7: bytes 0-3 = second operand
  const uint32_t hi = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, sel);  // codes 8-15
  const uint32_t m = ((c >> 3) & 0x01010101u) * 0xFFu;
  return (hi & m) | (lo & ~m);
}

// Q4_0: four nibbles, one in the low nibble of each byte of c (the other bits ignored), to the four int8 values
// nibble - 8, without borrows between bytes.
__device__ inline uint32_t q40_vals(uint32_t c) { return (((c & 0x0F0F0F0Fu) | 0x80808080u) - 0x08080808u) ^ 0x80808080u; }

// IQ3_XXS: the sign bits of values 8 l .. 8 l + 7 of a block from its word a: the 7-bit code at bit 7 l, and as the
// eighth bit the code's parity (ggml's ksigns_iq2xs, which the reference carries as a table: src/iq_tables.h).
__device__ inline uint32_t iq3xxs_signs8(uint32_t a, int l) {
  const uint32_t c = (a >> (7 * l)) & 127u;
  return c | ((__builtin_popcount(c) & 1u) << 7);
}

// Q3_K (device form): the four int8 values 4 k .. 4 k + 3 (k = 0..7) of a 32-value block from its words of low bits
// (D = D0 for k < 4, D1 above) and third bits H: the three bits - 4, no borrow between bytes.
__device__ inline uint32_t q3k_vals(uint32_t D, uint32_t H, int k) {
  const uint32_t v = ((D >> (2 * (k & 3))) & 0x03030303u) | (((H >> k) & 0x01010101u) << 2);
  return ((v | 0x80808080u) - 0x04040404u) ^ 0x80808080u;
}
// ... and the block's two scales - 32 from the header's three words (entry b at bit 12 b of the 96)
__device__ inline void q3k_scales(uint32_t s0, uint32_t s1, uint32_t s2, int b, int& sc0, int& sc1) {
  int a0, a1, m0, m1;
  q4k_scales_pair(s0, s1, s2, b >> 1, a0, a1, m0, m1);  // entries 2 (b / 2) and the next: (a0, m0), (a1, m1)
  sc0 = ((b & 1) ? a1 : a0) - 32;
  sc1 = ((b & 1) ? m1 : m0) - 32;
}

// MXFP4: four E2M1 codes, one in the low nibble of each byte of c, to the four int8 values of the format's table of
// doubled values (0 1 2 3 4 6 8 12 | 0 -1 -2 -3 -4 -6 -8 -12; reference src/quants.h:497): a byte permute per table
// half, the code's bit 3 picks between them (as iq4_lookup).
__device__ inline uint32_t mxfp4_lookup(uint32_t c) {
  const uint32_t sel = c & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);  // codes 0-7
  const uint32_t hi = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);  // codes 8-15
  const uint32_t m = ((c >> 3) & 0x01010101u) * 0xFFu;
  return (hi & m) | (lo & ~m);
}

// The types whose block is 16 bytes of nibbles and one scale (Q4_0, IQ4_NL, MXFP4) share every kernel path: the nibbles'
// values by the type's rule, the scale an f16 (Q4_0, IQ4_NL) or an E8M0 byte (MXFP4).
__host__ __device__ constexpr bool qt_nib16(int qt) { return qt == QT_Q4_0 || qt == QT_IQ4_NL || qt == QT_MXFP4; }
template <int QT>
__device__ inline uint32_t nib_vals(uint32_t c) {
  if constexpr (QT == QT_IQ4_NL) return iq4_lookup(c);
  else if constexpr (QT == QT_MXFP4) return mxfp4_lookup(c);
  else return q40_vals(c);
}
// (the scale plane lies where Q4_0's does, behind the nibbles: planes_q40(rows, nsb).d; an entry is 2 bytes or 1)
#define NIB16_SCALE_BYTES(QT) ((QT) == QT_MXFP4 ? 1 : 2)
// 2^(e - 128) of an E8M0 scale byte (e = 0, 1: the f32 subnormals 2^-128, 2^-127; reference src/quants.h:498-503)
__device__ inline float e8m0_half(uint32_t e) {
  e &= 0xFFu;
  return __builtin_bit_cast(float, e < 2 ? 0x00200000u << e : (e - 1) << 23);
}
// scale of block `blk` (counted over the whole plane) of a nibble type
template <int QT>
__device__ inline float nib16_scale(const uint8_t* plane, size_t blk) {
  if constexpr (QT == QT_MXFP4) return e8m0_half(plane[blk]);
  else return f16_bits_to_f32(*(const unsigned short*)(plane + blk * 2));
}

// IQ3_S: four magnitudes (bytes of a codebook entry g) with the four sign bits s4 (bit j: byte j is negative) applied:
// the bits are spread to the bytes' low bits by one multiply, and a byte is negated as (x ^ 0xFF) + 1 -- no carry
// leaves a byte, the magnitudes being 1..15.
__device__ inline uint32_t iq3s_signed4(uint32_t g, uint32_t s4) {
  const uint32_t m = (s4 * 0x00204081u) & 0x01010101u;
  return (g ^ (m * 0xFFu)) + m;
}

__device__ inline int dot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }
// The first product of a sum: the three-operand form with a constant 0 (the compiler picks the accumulate-in-place form
// for sdot4 and spends a move on clearing its register first).
__device__ inline int dot4_first(uint32_t a, uint32_t b) {
  int r;
  asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// x = x1 + x2 + x3 exactly, each piece a bf16 (x1 the top 8 significant bits by truncation, x2 the next 8, x3 the
// rest); w0 = x1 | x2 << 16, w1 = x3 (as bf16 bit patterns).
__device__ inline void split3(float x, uint32_t& w0, uint32_t& w1) {
  const uint32_t p1 = __float_as_uint(x) & 0xFFFF0000u;
  const float r1 = x - __uint_as_float(p1);
  const uint32_t p2 = __float_as_uint(r1) & 0xFFFF0000u;
  const float r2 = r1 - __uint_as_float(p2);
  w0 = (p1 >> 16) | p2;
  w1 = __float_as_uint(r2) >> 16;
}

// Sum over the 32 lanes of a half wave (lanes 0-31 and 32-63 separately), same value in every lane; a fixed tree,
// so results do not depend on anything but the inputs.
// The steps within a row of 16 lanes are data-parallel moves in the vector ALU (neighbour, other pair, other quad,
// other eight: after each step the lanes that have met hold the same sum, so taking the mirrored lane gives the sum of
// the other group); only the step between the two rows goes through the LDS crossbar.
template <int CTRL> __device__ inline float dpp_from(float v) {
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ inline float half_wave_sum(float v) {
  v += dpp_from<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_from<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_from<0x141>(v);  // row_half_mirror
  v += dpp_from<0x140>(v);  // row_mirror
  v += __shfl_xor(v, 16, 64);
  return v;
}
// Sum over each group of 32 (WIDE false) or all 64 lanes, valid in the LAST lane of the group only: the steps between
// rows of 16 are row broadcasts in the vector ALU too (lane 15 of a row added into the next row, lane 31 into the
// upper half), nothing goes through LDS.  A fixed tree as well.
template <bool WIDE> __device__ inline float group_sum_last(float v) {
  v += dpp_from<0xB1>(v);
  v += dpp_from<0x4E>(v);
  v += dpp_from<0x141>(v);
  v += dpp_from<0x140>(v);
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false));  // row_bcast15 -> rows 1, 3
  if constexpr (WIDE)
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xC, 0xF, false));  // row_bcast31 -> rows 2, 3
  return v;
}
// The output head's soft cap (the reference's -DSOFTCAP=c, zero/kernels/decode.cl:882-886): c * tanh(v / c) for c > 0,
// v itself for c = 0 (no cap).  c is the same for the whole launch.
__device__ inline float head_out(float v, float cap) { return cap > 0.0f ? cap * tanhf(v * (1.0f / cap)) : v; }
#endif
