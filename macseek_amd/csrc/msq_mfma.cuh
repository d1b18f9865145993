// MFMA building blocks for the multi-token paths (small-N matvec_n and the prefill grouped MoE GEMM).
//
// v_mfma_f32_16x16x32_{f16,bf16}: D[16 x 16] += A[16 x 32] . B[32 x 16], one wave.
//   A operand: lane l holds row  (l % 16), eight K positions 8 * (l / 16) .. + 7   (activations: row = token)
//   B operand: lane l holds col  (l % 16), the same eight K positions               (weights: col = weight row)
//   D operand: lane l holds col  (l % 16), rows 4 * (l / 16) + i, i = 0..3          (token, weight row)
// A and B only have to agree on which matrix column each K position means, so every format is free to pick the
// column order that makes its fragment cheap to decode (Frag::col_of).
//
// A fragment decoder turns the bytes of 8 weights of one row into 8 exact fp16 (or bf16) payloads plus an fp32 scale
// that is applied to the MFMA result, so weights are never rounded: weight = scale * payload (+ add, Q5_K only, which
// multiplies the per-token sum of the K step's activations).
#pragma once
#include "msq_device.cuh"

namespace msq {

typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));

constexpr int kMvnMaxSteps = 16;  // K steps (of 32 columns) whose activations one wave of the token-tile GEMM keeps in registers
constexpr int kMvnSubSteps = 8;   // K steps a wave of the small-N matvec fetches and multiplies at a time

__device__ __forceinline__ f4_t mfma_f16(const uint32_t a[4], const uint32_t b[4], f4_t c) {
  typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
  const u4_t av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8_t, av), __builtin_bit_cast(h8_t, bv), c, 0, 0, 0);
}
__device__ __forceinline__ f4_t mfma_bf16(const uint32_t a[4], const uint32_t b[4], f4_t c) {
  typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
  const u4_t av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, av), __builtin_bit_cast(bf8_t, bv), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t pk_add_f16(uint32_t a, uint32_t b) {
  const h2_t r = as_h2(a) + as_h2(b);
  return __builtin_bit_cast(uint32_t, r);
}
// float -> bf16 bits, round to nearest even (finite inputs)
__device__ __forceinline__ uint32_t bf16_rne(float f) {
  const uint32_t u = __builtin_bit_cast(uint32_t, f);
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// ================================================================================================ fragments
// Interface of a fragment decoder F (one K step = 32 matrix columns, chunk q = l / 16 of the step, 8 positions p):
//   BF16_MATH          payloads are bf16 (activations are then split into two bf16 terms) instead of fp16
//   HAS_ADD            weight = scale * payload + add
//   LDS_WORDS, fill_lds
//   col_of(q, p)       column (0..31 inside the step) that position p of chunk q stands for
//   get(row, step, q, tbl)   payloads of the 8 weights of weight row `row` (pointer to its first byte); the block
//                            formats split it into load_raw (the lane's bytes: loads only) and finish (table lookups
//                            and arithmetic), so that a kernel can request a step's bytes ahead of its arithmetic
struct FragOut {
  uint32_t h[4];
  float scale, add;
};

struct FragIQ1S {
  static constexpr bool BF16_MATH = false, HAS_ADD = false;
  static constexpr int WS_BYTES = 50;  // bytes of a row per 256 columns
  static constexpr int LDS_WORDS = MSQ_IQ1S_GRID_N * 4;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) { copy_words16(lds, g_tbl_iq1s.w, LDS_WORDS, tid, nt); }
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  struct Raw { uint32_t qh, qs, d; };
  template <class P>
  __device__ static Raw load_raw(P row, uint32_t step, uint32_t q) {
    const P b = row + (step >> 3) * 50u;
    const uint32_t ib = step & 7u;
    return {ld16(b + 34 + 2 * ib), ld8(b + 2 + 4 * ib + q), ld16(b)};
  }
  __device__ static FragOut finish(const Raw& r, uint32_t, uint32_t q, const uint32_t* tbl) {
    const uint32_t qh = r.qh;
    const uint32_t idx = r.qs | (((qh >> (3 * q)) & 7u) << 8);
    const uint4 g = ((const uint4*)tbl)[idx];
    const uint32_t delta2 = (qh & 0x8000u) ? 0xB000B000u : 0x30003000u;  // -0.125 / +0.125 in both halves
    FragOut o;
    o.h[0] = pk_add_f16(g.x, delta2); o.h[1] = pk_add_f16(g.y, delta2);  // grid + delta is exact in fp16
    o.h[2] = pk_add_f16(g.z, delta2); o.h[3] = pk_add_f16(g.w, delta2);
    o.scale = half_bits_to_float(r.d) * (float)(2u * ((qh >> 12) & 7u) + 1u);
    o.add = 0.f;
    return o;
  }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t* tbl) { return finish(load_raw(row, step, q), step, q, tbl); }
};

struct FragIQ2XXS {
  static constexpr bool BF16_MATH = false, HAS_ADD = false;
  static constexpr int WS_BYTES = 66;  // bytes of a row per 256 columns
  static constexpr int LDS_WORDS = MSQ_IQ2XXS_GRID_N * 4 + 128 * 4;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) { DecIQ2XXS::fill_lds(lds, tid, nt); }
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  template <class W32>
  struct Raw { W32 a1; uint32_t gi, d; };
  template <class P>
  __device__ static auto load_raw(P row, uint32_t step, uint32_t q) {
    const P b = row + (step >> 3) * 66u;
    const P a8 = b + 2 + 8 * (step & 7u);
    return Raw<decltype(ld32_raw(a8))>{ld32_raw(a8 + 4), ld8(a8 + q), ld16(b)};
  }
  template <class R>
  __device__ static FragOut finish(const R& r, uint32_t, uint32_t q, const uint32_t* tbl) {
    const uint32_t a1 = fix(r.a1);
    const uint4 g = ((const uint4*)tbl)[r.gi];
    const uint4 s = ((const uint4*)(tbl + MSQ_IQ2XXS_GRID_N * 4))[(a1 >> (7 * q)) & 127u];
    FragOut o;
    o.h[0] = g.x ^ s.x; o.h[1] = g.y ^ s.y; o.h[2] = g.z ^ s.z; o.h[3] = g.w ^ s.w;
    o.scale = half_bits_to_float(r.d) * (0.5f + (float)(a1 >> 28)) * 0.25f;
    o.add = 0.f;
    return o;
  }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t* tbl) { return finish(load_raw(row, step, q), step, q, tbl); }
};

struct FragQ8_0 {
  static constexpr bool BF16_MATH = false, HAS_ADD = false;
  static constexpr int WS_BYTES = 272;  // bytes of a row per 256 columns
  static constexpr int LDS_WORDS = 0;
  __device__ static void fill_lds(uint32_t*, int, int) {}
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  template <class W64>
  struct Raw { W64 v; uint32_t d; };
  template <class P>
  __device__ static auto load_raw(P row, uint32_t step, uint32_t q) {
    const P b = row + step * 34u;
    return Raw<decltype(ld64_raw(b))>{ld64_raw(b + 2 + 8 * q), ld16(b)};
  }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t* tbl) { return finish(load_raw(row, step, q), step, q, tbl); }
  template <class R>
  __device__ static FragOut finish(const R& r, uint32_t, uint32_t, const uint32_t*) {
    const u64_a2 v = fix(r.v);
    const uint32_t lo = v.x ^ 0x80808080u, hi = v.y ^ 0x80808080u;  // bytes become q + 128
    const uint32_t bias = 0xE480E480u;                              // -1152 in both halves
    FragOut o;
    o.h[0] = pk_add_f16(bytes01_to_h2_1024(lo), bias); o.h[1] = pk_add_f16(bytes23_to_h2_1024(lo), bias);
    o.h[2] = pk_add_f16(bytes01_to_h2_1024(hi), bias); o.h[3] = pk_add_f16(bytes23_to_h2_1024(hi), bias);
    o.scale = half_bits_to_float(r.d);
    o.add = 0.f;
    return o;
  }
};

// IQ4_NL: byte j of a block holds columns j (low nibble) and j + 16 (high nibble); chunk q takes bytes 4q .. 4q + 3, so
// its positions (2i, 2i + 1) stand for columns (4q + i, 4q + i + 16) and one table lookup per byte yields both.
struct FragIQ4NL {
  static constexpr bool BF16_MATH = false, HAS_ADD = false;
  static constexpr int WS_BYTES = 144;  // bytes of a row per 256 columns
  static constexpr int LDS_WORDS = 256;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) { copy_words16(lds, g_tbl_iq4nl.w, 256, tid, nt); }
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 4u * q + (p >> 1) + 16u * (p & 1u); }
  __device__ static uint32_t pos_of(uint32_t c) { return 8u * ((c & 15u) >> 2) + 2u * (c & 3u) + (c >> 4); }  // inverse of col_of
  template <class W32>
  struct Raw { W32 v; uint32_t d; };
  template <class P>
  __device__ static auto load_raw(P row, uint32_t step, uint32_t q) {
    const P b = row + step * 18u;
    return Raw<decltype(ld32_raw(b))>{ld32_raw(b + 2 + 4 * q), ld16(b)};
  }
  template <class R>
  __device__ static FragOut finish(const R& r, uint32_t, uint32_t, const uint32_t* tbl) {
    const uint32_t v = fix(r.v);
    FragOut o;
    o.h[0] = tbl[v & 0xFFu]; o.h[1] = tbl[(v >> 8) & 0xFFu]; o.h[2] = tbl[(v >> 16) & 0xFFu]; o.h[3] = tbl[v >> 24];
    o.scale = half_bits_to_float(r.d);
    o.add = 0.f;
    return o;
  }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t* tbl) { return finish(load_raw(row, step, q), step, q, tbl); }
};

// Q6_K: the 16-column scale groups are half a K step wide, so a step is issued as two MFMAs (chunks 0-1, chunks 2-3);
// get() returns the scale of the lane's own half and get_scales() both halves' scales of the lane's row.
struct FragQ6K {
  static constexpr bool BF16_MATH = false, HAS_ADD = false;
  static constexpr int WS_BYTES = 210;  // bytes of a row per 256 columns
  static constexpr int LDS_WORDS = 0;
  __device__ static void fill_lds(uint32_t*, int, int) {}
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t*) {
    const P b = row + (step >> 3) * 210u;
    const uint32_t e0 = 32u * (step & 7u) + 8u * q, h = e0 >> 7, k = (e0 & 127u) >> 5, l0 = e0 & 31u;
    const u64_a2 ql = ld64(b + 64 * h + 32 * (k & 1u) + l0), qh = ld64(b + 128 + 32 * h + l0);
    const uint32_t sh4 = 4u * (k >> 1), sh2 = 2u * k;
    const uint32_t q0 = ((ql.x >> sh4) & 0x0F0F0F0Fu) | (((qh.x >> sh2) & 0x03030303u) << 4);
    const uint32_t q1 = ((ql.y >> sh4) & 0x0F0F0F0Fu) | (((qh.y >> sh2) & 0x03030303u) << 4);
    const uint32_t bias = 0xE420E420u;  // -1056 = -(1024 + 32) in both halves
    FragOut o;
    o.h[0] = pk_add_f16(bytes01_to_h2_1024(q0), bias); o.h[1] = pk_add_f16(bytes23_to_h2_1024(q0), bias);
    o.h[2] = pk_add_f16(bytes01_to_h2_1024(q1), bias); o.h[3] = pk_add_f16(bytes23_to_h2_1024(q1), bias);
    o.scale = 0.f;
    o.add = 0.f;
    return o;
  }
  template <class W64>
  struct Raw { W64 ql, qh; uint32_t sc, d; };
  template <class P>
  __device__ static auto load_raw(P row, uint32_t step, uint32_t q) {
    const P b = row + (step >> 3) * 210u;
    const uint32_t e0 = 32u * (step & 7u) + 8u * q, h = e0 >> 7, k = (e0 & 127u) >> 5, l0 = e0 & 31u;
    return Raw<decltype(ld64_raw(b))>{ld64_raw(b + 64 * h + 32 * (k & 1u) + l0), ld64_raw(b + 128 + 32 * h + l0),
                                      ld16(b + 192 + 8 * h + 2 * k), ld16(b + 208)};
  }
  // (the scale of the lane's own half of the step: chunks 0-1 the first 16 columns, chunks 2-3 the second)
  template <class R>
  __device__ static FragOut finish(const R& r, uint32_t step, uint32_t q, const uint32_t*) {
    const uint32_t k = step & 3u;
    const uint32_t sh4 = 4u * (k >> 1), sh2 = 2u * k;
    const u64_a2 ql = fix(r.ql), qh = fix(r.qh);
    const uint32_t q0 = ((ql.x >> sh4) & 0x0F0F0F0Fu) | (((qh.x >> sh2) & 0x03030303u) << 4);
    const uint32_t q1 = ((ql.y >> sh4) & 0x0F0F0F0Fu) | (((qh.y >> sh2) & 0x03030303u) << 4);
    const uint32_t bias = 0xE420E420u;  // -1056 = -(1024 + 32) in both halves
    FragOut o;
    o.h[0] = pk_add_f16(bytes01_to_h2_1024(q0), bias); o.h[1] = pk_add_f16(bytes23_to_h2_1024(q0), bias);
    o.h[2] = pk_add_f16(bytes01_to_h2_1024(q1), bias); o.h[3] = pk_add_f16(bytes23_to_h2_1024(q1), bias);
    o.scale = half_bits_to_float(r.d) * (float)(int)(int8_t)(q < 2 ? r.sc & 0xFFu : r.sc >> 8);
    o.add = 0.f;
    return o;
  }
  template <class P>
  __device__ static void get_scales(P row, uint32_t step, float& sa, float& sb) {
    const P b = row + (step >> 3) * 210u;
    const uint32_t e0 = 32u * (step & 7u), h = e0 >> 7, k = (e0 & 127u) >> 5;
    const uint32_t sc = ld16(b + 192 + 8 * h + 2 * k);
    const float d = half_bits_to_float(ld16(b + 208));
    sa = d * (float)(int)(int8_t)(sc & 0xFFu);
    sb = d * (float)(int)(int8_t)(sc >> 8);
  }
};

struct FragQ5K {
  static constexpr bool BF16_MATH = false, HAS_ADD = true;
  static constexpr int WS_BYTES = 176;  // bytes of a row per 256 columns
  static constexpr int LDS_WORDS = 0;
  __device__ static void fill_lds(uint32_t*, int, int) {}
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  template <class W64, class W128>
  struct Raw { W64 ql, qh; W128 hdr; };  // hdr: d | dmin, then the 12 scale bytes
  template <class P>
  __device__ static auto load_raw(P row, uint32_t step, uint32_t q) {
    const P b = row + (step >> 3) * 176u;
    const uint32_t g = (step & 7u) >> 1, l0 = 8u * q;
    return Raw<decltype(ld64_raw(b)), decltype(ld128_raw(b))>{ld64_raw(b + 48 + 32 * g + l0), ld64_raw(b + 16 + l0), ld128_raw(b)};
  }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t* tbl) { return finish(load_raw(row, step, q), step, q, tbl); }
  template <class R>
  __device__ static FragOut finish(const R& r, uint32_t step, uint32_t, const uint32_t*) {
    const uint32_t is = step & 7u, run = is & 1u;
    const u64_a2 ql = fix(r.ql), qh = fix(r.qh);
    const u128_a2 hdr = fix(r.hdr);
    const uint32_t q0 = ((ql.x >> (4 * run)) & 0x0F0F0F0Fu) | (((qh.x >> is) & 0x01010101u) << 4);
    const uint32_t q1 = ((ql.y >> (4 * run)) & 0x0F0F0F0Fu) | (((qh.y >> is) & 0x01010101u) << 4);
    const uint32_t bias = 0xE400E400u;  // -1024 in both halves
    // (all 12 scale bytes were fetched: a load inside a branch makes the waits that follow conservative)
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    auto byte = [&](uint32_t i) { const uint32_t w = i < 4 ? s0 : i < 8 ? s1 : s2; return (w >> (8 * (i & 3u))) & 0xFFu; };
    uint32_t sc, mn;
    if (is < 4) { sc = byte(is) & 63u; mn = byte(is + 4) & 63u; }
    else { sc = (byte(is + 4) & 0xFu) | ((byte(is - 4) >> 6) << 4); mn = (byte(is + 4) >> 4) | ((byte(is) >> 6) << 4); }
    const uint32_t dd = hdr.x;
    FragOut o;
    o.h[0] = pk_add_f16(bytes01_to_h2_1024(q0), bias); o.h[1] = pk_add_f16(bytes23_to_h2_1024(q0), bias);
    o.h[2] = pk_add_f16(bytes01_to_h2_1024(q1), bias); o.h[3] = pk_add_f16(bytes23_to_h2_1024(q1), bias);
    o.scale = half_bits_to_float(dd & 0xFFFFu) * (float)sc;
    o.add = -(half_bits_to_float(dd >> 16) * (float)mn);
    return o;
  }
};

template <int QT>  // MSQ_F16 or MSQ_BF16
struct FragDense16 {
  static constexpr bool BF16_MATH = QT == MSQ_BF16, HAS_ADD = false, PLAIN = true;  // PLAIN: the payload is the weight
  static constexpr int LDS_WORDS = 0;
  __device__ static void fill_lds(uint32_t*, int, int) {}
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t*) {
    const u128_a2 v = ld128(row + 64u * step + 16u * q);
    FragOut o;
    o.h[0] = v.x; o.h[1] = v.y; o.h[2] = v.z; o.h[3] = v.w;
    o.scale = 1.f;
    o.add = 0.f;
    return o;
  }
};

// ================================================================================================ block fragments
// For the 256-weight codebook formats the large-token GEMM uses a second decomposition: the payload is the whole weight,
// scale included, as fp16 (the reference's prefill kernels feed their matrix units dequantized fp16 tiles too; they
// round d * scale * grid once, src/kernels/quant_moe_prefill.metal:137-167, where finish() below rounds twice: the
// sub-block scale to fp16, then its product with the grid value, 2^-11 relative per weight at worst instead of
// 2^-12; the scale in fp32 would cost a second multiply per register), so a wave accumulates
// all of K in the matrix cores without touching the accumulators in between. Lane (row n, chunk q) owns the sub-blocks 2 q and 2 q + 1 of its row's block
// (16 contiguous bytes of IQ2_XXS), so no lane loads a byte twice; step j (0..7) of a block therefore covers, for chunk
// q, the 8 columns col_of(q, j) .. + 7 of the block, and the activation operand is read with the same mapping.
//   Raw / load(block pointer, q)    the lane's bytes of one block
//   lookup(raw, j, tbl, col)        table reads of step j (col = lane % 16), issued ahead of their use
//   finish(raw, j, look, h)         payloads of step j
__device__ __forceinline__ uint32_t pk_mul_f16(uint32_t a, uint32_t b) {
  const h2_t r = as_h2(a) * as_h2(b);
  return __builtin_bit_cast(uint32_t, r);
}
// both halves = (fp16)v for an integer 0 <= v < 1024, without a conversion: 0x6400 | v is 1024 + v
__device__ __forceinline__ uint32_t pk_small_int_f16(uint32_t v) {
  return pk_add_f16(0x64006400u | v | (v << 16), 0xE400E400u);
}
// N dwords from a global address that is only 2-byte aligned, fetched with 4-byte-aligned loads: wide loads that are
// not dword aligned run at about a third of the rate of aligned ones. N aligned dwords plus the one that follows (the
// last one again when the address is aligned, so nothing past the data is touched), then a funnel shift.
template <int N>
__device__ __forceinline__ void ld_dwords_2aligned(gptr_t p, uint32_t (&out)[N]) {
  typedef uint32_t __attribute__((ext_vector_type(N), aligned(4))) vec_t;
  const uintptr_t a = (uintptr_t)p;
  const uint32_t odd = (uint32_t)a & 2u;
  const MSQ_GLOBAL uint32_t* w = (const MSQ_GLOBAL uint32_t*)(a - odd);
  const vec_t v = *(const MSQ_GLOBAL vec_t*)w;
  const uint32_t tail = w[odd ? N : N - 1];
#pragma unroll
  for (int i = 0; i < N; i++) out[i] = __builtin_amdgcn_alignbit(i + 1 < N ? v[i + 1] : tail, v[i], odd * 8u);
}
__device__ __forceinline__ uint32_t blk_col_of(uint32_t q, uint32_t j) { return 64u * q + 32u * (j >> 2) + 8u * (j & 3u); }

// IQ2_XXS keeps 16 copies of its two small tables in LDS, copy c in the 16-byte bank column c of each 256-byte row:
// a 16-lane group whose lanes read "their" column (c = lane % 16) touches every bank exactly once whatever the
// entries are, so the random lookups run at the conflict-free rate.
struct BlkIQ2XXS {
  static constexpr int LDS_WORDS = (MSQ_IQ2XXS_GRID_N + 128) * 16 * 4, BLOCK_BYTES = 66;
  // the sign table comes first: both table bases then fit the 16-bit offset field of the LDS instructions (signs at 0,
  // grid at 32 KB), and a lookup address is one v_and_or of the entry index and the lane's column
  static constexpr uint32_t GRID_AT = 128u * 256u;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) {
    const uint4* grid = (const uint4*)g_tbl_iq2xxs.w;
    const uint4* sign = (const uint4*)g_tbl_sign.w;
    uint4* dst = (uint4*)lds;
    for (int i = tid; i < (MSQ_IQ2XXS_GRID_N + 128) * 16; i += nt) {
      const int e = i >> 4;
      dst[i] = e < 128 ? sign[e] : grid[e - 128];
    }
  }
  struct Raw { uint32_t w[4]; uint32_t d; };  // {a0, a1} of sub-block 2 q, then of 2 q + 1; fp16 bits of d
  __device__ static Raw load(gptr_t blk, uint32_t q) {
    Raw r;
    ld_dwords_2aligned<4>(blk + 2 + 16 * q, r.w);
    r.d = ld16(blk);
    return r;
  }
  struct Look { uint4 g, s; };
  // byte offsets in the replicated tables: entry << 8 | column << 4
  __device__ static Look lookup(const Raw& r, int j, const uint32_t* tbl, uint32_t col) {
    const uint32_t a0 = r.w[2 * (j >> 2)], a1 = r.w[2 * (j >> 2) + 1];
    const int l = j & 3;
    const uint32_t cg = col << 4;
    const uint32_t g8 = l == 0 ? a0 << 8 : l == 1 ? a0 : a0 >> (8 * l - 8);    // grid index byte at bits 8..15
    const uint32_t s8 = 7 * l < 8 ? a1 << (8 - 7 * l) : a1 >> (7 * l - 8);     // sign index at bits 8..14
    const uint8_t* t8 = (const uint8_t*)tbl;
    return {*(const uint4*)(t8 + GRID_AT + ((g8 & 0xFF00u) | cg)), *(const uint4*)(t8 + ((s8 & 0x7F00u) | cg))};
  }
  // weight = fp16(fp16(d (2 s + 1) / 8) * (+-grid)): the whole scale rides in the payload, rounded to fp16 before the
  // multiply (the reference's tile rounds the fp32 product once, src/kernels/quant_moe_prefill.metal:153-167)
  __device__ static void finish(const Raw& r, int j, const Look& k, uint32_t (&h)[4]) {
    const uint32_t a1 = r.w[2 * (j >> 2) + 1];
    const float m = (half_bits_to_float(r.d) * 0.125f) * (float)(((a1 >> 27) & 0x1Eu) | 1u);
    const uint32_t m2 = pack_h2(m, m);
    h[0] = pk_mul_f16(k.g.x ^ k.s.x, m2); h[1] = pk_mul_f16(k.g.y ^ k.s.y, m2);
    h[2] = pk_mul_f16(k.g.z ^ k.s.z, m2); h[3] = pk_mul_f16(k.g.w ^ k.s.w, m2);
  }
};

struct BlkIQ1S {
  static constexpr int LDS_WORDS = FragIQ1S::LDS_WORDS, BLOCK_BYTES = 50;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) { FragIQ1S::fill_lds(lds, tid, nt); }
  struct Raw { uint32_t qs[2]; uint32_t qh; uint32_t d; };  // qs bytes 8 q .. 8 q + 7; qh[2 q] | qh[2 q + 1] << 16
  __device__ static Raw load(gptr_t blk, uint32_t q) {
    Raw r;
    uint32_t qh[1];
    ld_dwords_2aligned<2>(blk + 2 + 8 * q, r.qs);
    ld_dwords_2aligned<1>(blk + 34 + 4 * q, qh);
    r.qh = qh[0];
    r.d = ld16(blk);
    return r;
  }
  struct Look { uint4 g; };
  __device__ static Look lookup(const Raw& r, int j, const uint32_t* tbl, uint32_t) {
    const uint32_t qs = r.qs[j >> 2], qh = (j >> 2) ? r.qh >> 16 : r.qh & 0xFFFFu;
    const int l = j & 3;
    return {((const uint4*)tbl)[((qs >> (8 * l)) & 0xFFu) | (((qh >> (3 * l)) & 7u) << 8)]};
  }
  // weight = fp16(fp16(d (2 s + 1)) * (grid + delta)): scale rounded to fp16, product rounded again (the reference's
  // tile rounds the fp32 product once, src/kernels/quant_moe_prefill.metal:137-147)
  __device__ static void finish(const Raw& r, int j, const Look& k, uint32_t (&h)[4]) {
    const uint32_t qh = (j >> 2) ? r.qh >> 16 : r.qh & 0xFFFFu;
    const uint32_t d2 = (qh & 0x8000u) ? 0xB000B000u : 0x30003000u;          // -+ 1/8 in both halves
    const float m = half_bits_to_float(r.d) * (float)(((qh >> 11) & 0xEu) | 1u);
    const uint32_t m2 = pack_h2(m, m);
    h[0] = pk_mul_f16(pk_add_f16(k.g.x, d2), m2); h[1] = pk_mul_f16(pk_add_f16(k.g.y, d2), m2);
    h[2] = pk_mul_f16(pk_add_f16(k.g.z, d2), m2); h[3] = pk_mul_f16(pk_add_f16(k.g.w, d2), m2);
  }
};

}  // namespace msq
