// Device-side building blocks for gfx950 (wave64): codebook tables, unaligned block loads, DPP wave reduction and the
// per-format block decoders used by the decode (n = 1) kernels.
//
// Block byte layouts and element order follow the GGUF formats as restated by the reference's CPU dequantizer
// (tests/ref/dequant.cpp:34-120). Lane/unit mappings are this library's own: one lane owns a UNIT-column slice of a
// row (32 columns for the block formats) and keeps the matching activations in registers as fp16 pairs, so a row
// costs one packed dot (v_dot2_f32_f16) per two weights plus the decode.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iq_codebooks.h"
#include "msq_types.h"

namespace msq {

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// ------------------------------------------------------------------------------------------------ constant tables
// fp16 images of the codebooks, expanded at compile time from the base-3 packed form.
// 8 halves (-1, 0, +1) per entry, then sixteen {2 s + 1, -+ (2 s + 1) / 8} float pairs indexed by the top four bits of qh
struct TblIQ1S { uint32_t w[MSQ_IQ1S_GRID_N * 4 + 32]; };
struct TblIQ2XXS { uint32_t w[MSQ_IQ2XXS_GRID_N * 4]; };  // 8 halves (8, 25, 43) per entry
struct TblSign { uint32_t w[128 * 4]; };                  // 8 fp16 sign-bit masks per 7-bit sign index
struct TblIQ4NL { uint32_t w[256]; };                     // byte -> {half(kv[lo nibble]), half(kv[hi nibble])}

constexpr uint16_t half_of_small_int(int v) {  // exact fp16 bits of an integer |v| < 2048
  if (v == 0) return 0;
  const uint16_t s = v < 0 ? 0x8000 : 0;
  unsigned a = v < 0 ? (unsigned)-v : (unsigned)v;
  int e = 0;
  while ((a >> (e + 1)) != 0) e++;
  const unsigned man = (a << (10 - e)) & 0x3FFu;
  return (uint16_t)(s | (unsigned)((e + 15) << 10) | man);
}
constexpr TblIQ1S make_iq1s() {
  TblIQ1S t{};
  constexpr uint16_t hv[3] = {0xBC00, 0x0000, 0x3C00};
  for (int i = 0; i < MSQ_IQ1S_GRID_N; i++) {
    unsigned c = msq_iq1s_code[i];
    for (int j = 0; j < 4; j++) {
      const uint32_t lo = hv[c % 3]; c /= 3;
      const uint32_t hi = hv[c % 3]; c /= 3;
      t.w[4 * i + j] = lo | (hi << 16);
    }
  }
  // the sub-block factors of a unit, ready made: entry k = qh >> 12 (bit 3: sign of delta, bits 0..2: s) holds the
  // floats 2 s + 1 and (k & 8 ? -0.125 : +0.125) * (2 s + 1), both exact
  for (int k = 0; k < 16; k++) {
    const int f = 2 * (k & 7) + 1;  // 1, 3, .. 15
    int e = 0;
    while ((f >> (e + 1)) != 0) e++;
    const uint32_t fb = ((uint32_t)(e + 127) << 23) | (((uint32_t)f << (23 - e)) & 0x7FFFFFu);  // float bits of f
    t.w[MSQ_IQ1S_GRID_N * 4 + 2 * k] = fb;
    t.w[MSQ_IQ1S_GRID_N * 4 + 2 * k + 1] = (fb - (3u << 23)) | ((k & 8) ? 0x80000000u : 0u);  // f / 8 with delta's sign
  }
  return t;
}
constexpr TblIQ2XXS make_iq2xxs() {
  TblIQ2XXS t{};
  constexpr uint16_t hv[3] = {half_of_small_int(8), half_of_small_int(25), half_of_small_int(43)};
  for (int i = 0; i < MSQ_IQ2XXS_GRID_N; i++) {
    unsigned c = msq_iq2xxs_code[i];
    for (int j = 0; j < 4; j++) {
      const uint32_t lo = hv[c % 3]; c /= 3;
      const uint32_t hi = hv[c % 3]; c /= 3;
      t.w[4 * i + j] = lo | (hi << 16);
    }
  }
  return t;
}
constexpr TblSign make_sign() {  // ksigns_iq2xs[i] = i | parity(i) << 7; bit j set => element j negative
  TblSign t{};
  for (int i = 0; i < 128; i++) {
    int par = 0;
    for (int b = 0; b < 7; b++) par ^= (i >> b) & 1;
    const unsigned s = (unsigned)i | ((unsigned)par << 7);
    for (int j = 0; j < 4; j++)
      t.w[4 * i + j] = ((s >> (2 * j)) & 1 ? 0x8000u : 0u) | ((s >> (2 * j + 1)) & 1 ? 0x80000000u : 0u);
  }
  return t;
}
constexpr int kIQ4NLValues[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
constexpr TblIQ4NL make_iq4nl() {
  TblIQ4NL t{};
  for (int b = 0; b < 256; b++)
    t.w[b] = (uint32_t)half_of_small_int(kIQ4NLValues[b & 15]) | ((uint32_t)half_of_small_int(kIQ4NLValues[b >> 4]) << 16);
  return t;
}

__device__ __attribute__((aligned(16))) const TblIQ1S g_tbl_iq1s = make_iq1s();
__device__ __attribute__((aligned(16))) const TblIQ2XXS g_tbl_iq2xxs = make_iq2xxs();
__device__ __attribute__((aligned(16))) const TblSign g_tbl_sign = make_sign();
__device__ __attribute__((aligned(16))) const TblIQ4NL g_tbl_iq4nl = make_iq4nl();

// ------------------------------------------------------------------------------------------------ loads
// GGUF blocks are only 2-byte aligned (34/50/66/210-byte blocks, matrices placed at 4-byte offsets); gfx950 global
// loads accept any alignment, so wider-than-alignment loads are expressed through under-aligned types.
typedef uint32_t __attribute__((aligned(2), may_alias)) u32_a2;
struct __attribute__((packed, aligned(2))) u64_a2 { uint32_t x, y; };
struct __attribute__((packed, aligned(2))) u128_a2 { uint32_t x, y, z, w; };

typedef uint32_t __attribute__((ext_vector_type(2), aligned(2))) u32x2_a2;
typedef uint32_t __attribute__((ext_vector_type(4), aligned(2))) u32x4_a2;

// Weight pointers that reach a kernel through a table or a struct are "generic" to the compiler, and generic loads are
// FLAT instructions: they count against the LDS counter as well, so every wait for a table lookup would also wait for
// the weight prefetches in flight. Such pointers are therefore cast to the global address space (gptr_t) once, and
// the byte loaders exist for both kinds of pointer.
#define MSQ_GLOBAL __attribute__((address_space(1)))
typedef const MSQ_GLOBAL uint8_t* gptr_t;
__device__ __forceinline__ gptr_t as_global(const void* p) { return (gptr_t)p; }

// Range-checked buffer loads: the descriptor covers `bytes` bytes at `base`; a load whose offset falls outside returns
// zero without touching memory. A pipelined loop can thus issue its prefetches unconditionally (an empty descriptor for
// the rows past the end), which keeps the number of loads in flight known at every wait.
typedef uint32_t __attribute__((ext_vector_type(4))) u32x4;
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint32_t buf_ld16(rsrc_t r, uint32_t voff, uint32_t soff) {
  return (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, (int)voff, (int)soff, 0);
}
__device__ __forceinline__ uint32_t buf_ld32(rsrc_t r, uint32_t voff, uint32_t soff) {
  return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0);
}
__device__ __forceinline__ u64_a2 buf_ld64(rsrc_t r, uint32_t voff, uint32_t soff) {
  const auto v = __builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, (int)soff, 0);
  return {(uint32_t)v[0], (uint32_t)v[1]};
}

__device__ __forceinline__ u128_a2 buf_ld128(rsrc_t r, uint32_t voff, uint32_t soff) {
  const auto v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
  return {(uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]};
}
__device__ __forceinline__ u32x4 buf_ld128v(rsrc_t r, uint32_t voff, uint32_t soff) {
  const auto v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
  return u32x4{(uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]};
}
// A weight row reached through a buffer descriptor, in the shape of a pointer for the decoders' load() functions
// (p + bytes, ld16 .. ld128): rs covers a run of rows, soff is the row's byte offset in it -- wave-uniform, so it travels
// in a scalar register -- and voff the lane's byte offset inside the row, a loop constant. A row's loads then cost no
// vector arithmetic (a 64-bit pointer per lane costs a multiply-add and an addition per load and row).
struct BufRow {
  rsrc_t rs;
  uint32_t soff, voff;
  __device__ __forceinline__ BufRow operator+(uint32_t o) const { return {rs, soff, voff + o}; }
};
__device__ __forceinline__ uint32_t ld16(const BufRow& p) { return buf_ld16(p.rs, p.voff, p.soff); }
__device__ __forceinline__ uint32_t ld32(const BufRow& p) { return buf_ld32(p.rs, p.voff, p.soff); }
__device__ __forceinline__ u64_a2 ld64(const BufRow& p) { return buf_ld64(p.rs, p.voff, p.soff); }
__device__ __forceinline__ u128_a2 ld128(const BufRow& p) { return buf_ld128(p.rs, p.voff, p.soff); }

// A weight row whose bytes a wave holds in LDS (see mv_tok_kernel): `base` is the wave's 16-byte-aligned buffer, at + sh
// the byte offset in it, only 2-byte aligned like the blocks themselves, kept as its aligned part and its low two bits.
// LDS reads want aligned addresses: a load reads the aligned words that hold its bytes and shifts them into place.
// (Two fields: the offsets a decoder adds behind the block's are multiples of four, which the compiler can see, so
// that the split is made once per block and not once per load.)
struct LdsRow {
  const uint8_t* base;
  uint32_t at, sh;
  __device__ __forceinline__ static LdsRow of(const uint8_t* base, uint32_t off) { return {base, off & ~3u, off & 3u}; }
  __device__ __forceinline__ LdsRow operator+(uint32_t o) const {
    const uint32_t t = sh + o;
    return {base, at + (t & ~3u), t & 3u};
  }
};
__device__ __forceinline__ uint32_t ld8(const LdsRow& p) { return *(p.base + p.at + p.sh); }
__device__ __forceinline__ uint32_t ld16(const LdsRow& p) { return *(const uint16_t*)(p.base + p.at + p.sh); }
__device__ __forceinline__ uint32_t ld32(const LdsRow& p) {
  const uint32_t* q = (const uint32_t*)(p.base + p.at);
  return __builtin_amdgcn_alignbyte(q[1], q[0], p.sh);
}
__device__ __forceinline__ u64_a2 ld64(const LdsRow& p) {
  const uint32_t* q = (const uint32_t*)(p.base + p.at);
  const uint32_t d0 = q[0], d1 = q[1], d2 = q[2];
  return {__builtin_amdgcn_alignbyte(d1, d0, p.sh), __builtin_amdgcn_alignbyte(d2, d1, p.sh)};
}
__device__ __forceinline__ u128_a2 ld128(const LdsRow& p) {
  const uint32_t* q = (const uint32_t*)(p.base + p.at);
  const uint32_t d0 = q[0], d1 = q[1], d2 = q[2], d3 = q[3], d4 = q[4];
  return {__builtin_amdgcn_alignbyte(d1, d0, p.sh), __builtin_amdgcn_alignbyte(d2, d1, p.sh), __builtin_amdgcn_alignbyte(d3, d2, p.sh),
          __builtin_amdgcn_alignbyte(d4, d3, p.sh)};
}

// Loads in two parts, for kernels that request bytes ahead of the arithmetic on them: ldN_raw(p) only issues the
// loads, fix() puts the bytes in place. For memory pointers the first part does everything; for LDS rows the aligned
// words are read first and shifted when they are used (a shift right behind its read would wait for the read).
struct Lds32Raw { uint32_t d0, d1, sh; };
struct Lds64Raw { uint32_t d0, d1, d2, sh; };
struct Lds128Raw { uint32_t d0, d1, d2, d3, d4, sh; };
__device__ __forceinline__ Lds32Raw ld32_raw(const LdsRow& p) {
  const uint32_t* q = (const uint32_t*)(p.base + p.at);
  return {q[0], q[1], p.sh};
}
__device__ __forceinline__ Lds64Raw ld64_raw(const LdsRow& p) {
  const uint32_t* q = (const uint32_t*)(p.base + p.at);
  return {q[0], q[1], q[2], p.sh};
}
__device__ __forceinline__ Lds128Raw ld128_raw(const LdsRow& p) {
  const uint32_t* q = (const uint32_t*)(p.base + p.at);
  return {q[0], q[1], q[2], q[3], q[4], p.sh};
}
__device__ __forceinline__ uint32_t fix(const Lds32Raw& r) { return __builtin_amdgcn_alignbyte(r.d1, r.d0, r.sh); }
__device__ __forceinline__ u64_a2 fix(const Lds64Raw& r) {
  return {__builtin_amdgcn_alignbyte(r.d1, r.d0, r.sh), __builtin_amdgcn_alignbyte(r.d2, r.d1, r.sh)};
}
__device__ __forceinline__ u128_a2 fix(const Lds128Raw& r) {
  return {__builtin_amdgcn_alignbyte(r.d1, r.d0, r.sh), __builtin_amdgcn_alignbyte(r.d2, r.d1, r.sh),
          __builtin_amdgcn_alignbyte(r.d3, r.d2, r.sh), __builtin_amdgcn_alignbyte(r.d4, r.d3, r.sh)};
}
__device__ __forceinline__ uint32_t fix(uint32_t v) { return v; }
__device__ __forceinline__ u64_a2 fix(const u64_a2& v) { return v; }
__device__ __forceinline__ u128_a2 fix(const u128_a2& v) { return v; }

#define MSQ_LOADERS(AS)                                                                                               \
  __device__ __forceinline__ uint32_t ld8(const AS uint8_t* p) { return *p; }                                         \
  __device__ __forceinline__ uint32_t ld16(const AS uint8_t* p) { return *(const AS uint16_t*)p; }                    \
  __device__ __forceinline__ uint32_t ld32(const AS uint8_t* p) { return *(const AS u32_a2*)p; }                      \
  __device__ __forceinline__ u64_a2 ld64(const AS uint8_t* p) {                                                       \
    const u32x2_a2 v = *(const AS u32x2_a2*)p;                                                                        \
    return {v.x, v.y};                                                                                                \
  }                                                                                                                   \
  __device__ __forceinline__ u128_a2 ld128(const AS uint8_t* p) {                                                     \
    const u32x4_a2 v = *(const AS u32x4_a2*)p;                                                                        \
    return {v.x, v.y, v.z, v.w};                                                                                      \
  }                                                                                                                   \
  __device__ __forceinline__ uint32_t ld32_raw(const AS uint8_t* p) { return ld32(p); }                               \
  __device__ __forceinline__ u64_a2 ld64_raw(const AS uint8_t* p) { return ld64(p); }                                 \
  __device__ __forceinline__ u128_a2 ld128_raw(const AS uint8_t* p) { return ld128(p); }
MSQ_LOADERS()
MSQ_LOADERS(MSQ_GLOBAL)
#undef MSQ_LOADERS

__device__ __forceinline__ float half_bits_to_float(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}
__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __builtin_bit_cast(float, b << 16); }
__device__ __forceinline__ h2_t as_h2(uint32_t v) { return __builtin_bit_cast(h2_t, v); }
__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
  h2_t v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
  return __builtin_amdgcn_fdot2(as_h2(w), as_h2(x), acc, false);
}
// bytes b0,b1 (sel_lo) or b2,b3 (sel_hi) of q become the halves 1024 + b (0x6400 | b)
__device__ __forceinline__ uint32_t bytes01_to_h2_1024(uint32_t q) { return __builtin_amdgcn_perm(0x64646464u, q, 0x04010400u); }
__device__ __forceinline__ uint32_t bytes23_to_h2_1024(uint32_t q) { return __builtin_amdgcn_perm(0x64646464u, q, 0x04030402u); }

// ------------------------------------------------------------------------------------------------ wave reduction
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false);
  return v + __builtin_bit_cast(float, moved);
}
// Sum over the 64 lanes of a wave; the total is returned in every lane (broadcast through a scalar register).
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);        // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);        // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);       // row_half_mirror
  v = dpp_add<0x140>(v);       // row_mirror: every lane of a 16-lane row holds the row sum
  v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
  v = dpp_add<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3: lane 63 holds the total
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Transposed partial reduction: N independent per-lane values (N = 1, 2, 4 or 8) are folded over the 8-lane group of
// each lane in three DPP steps (lane i <-> 7 - i, then i <-> i ^ 1, then i <-> i ^ 2). A step that still has several
// values to tell apart halves their number: a lane keeps the half its lane bit selects and receives its partner's
// contribution to that half. Afterwards v[0] of lane l holds value number group8_sel<N>(l) summed over l's group.
// This costs three ops per value pair instead of six full-wave steps per value; callers add the eight group sums of
// a wave (and the K-split waves) in LDS in a fixed order.
template <int CTRL>
__device__ __forceinline__ float dpp_fold(float keep, float send) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, send), CTRL, 0xF, 0xF, false);
  return keep + __builtin_bit_cast(float, moved);
}
template <int N>
__device__ __forceinline__ void group8_fold(float* v, uint32_t lane) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8, "group8_fold: N must be 1, 2, 4 or 8");
  const bool b0 = lane & 1u, b1 = lane & 2u, b2 = lane & 4u;
  constexpr int N1 = N >= 2 ? N / 2 : 1, N2 = N >= 4 ? N / 4 : 1;
  // step 1: partner 7 - i (row_half_mirror) differs in bit 2
#pragma unroll
  for (int i = 0; i < N1; i++) {
    if constexpr (N >= 2) { const float lo = v[i], hi = v[i + N1]; v[i] = dpp_fold<0x141>(b2 ? hi : lo, b2 ? lo : hi); }
    else v[i] = dpp_fold<0x141>(v[i], v[i]);
  }
  // step 2: partner i ^ 1 (quad_perm [1,0,3,2]) differs in bit 0
#pragma unroll
  for (int i = 0; i < N2; i++) {
    if constexpr (N >= 4) { const float lo = v[i], hi = v[i + N2]; v[i] = dpp_fold<0xB1>(b0 ? hi : lo, b0 ? lo : hi); }
    else v[i] = dpp_fold<0xB1>(v[i], v[i]);
  }
  // step 3: partner i ^ 2 (quad_perm [2,3,0,1]) differs in bit 1
  if constexpr (N >= 8) { const float lo = v[0], hi = v[1]; v[0] = dpp_fold<0x4E>(b1 ? hi : lo, b1 ? lo : hi); }
  else v[0] = dpp_fold<0x4E>(v[0], v[0]);
}
// group8_fold followed by one more step (lane i <-> i ^ 8, row_ror:8): v[0] holds the sum over the lane's 16-lane row.
template <int N>
__device__ __forceinline__ void row16_fold(float* v, uint32_t lane) {
  group8_fold<N>(v, lane);
  v[0] = dpp_fold<0x128>(v[0], v[0]);
}
// number of the value lane l holds after group8_fold<N>
template <int N>
__device__ __forceinline__ uint32_t group8_sel(uint32_t lane) {
  uint32_t s = 0;
  if (N >= 2) s += ((lane >> 2) & 1u) * (N / 2);
  if (N >= 4) s += (lane & 1u) * (N / 4);
  if (N >= 8) s += ((lane >> 1) & 1u) * (N / 8);
  return s;
}

// Sum of n partial results p[0], p[stride], ... in that order. Eight are read before the first is added: read and
// added one at a time, the loop is a chain of LDS latencies (28 of them per output row in the MoE down kernel).
__device__ __forceinline__ float sum_in_order(const float* p, uint32_t n, uint32_t stride = 1) {
  float s = 0.f;
  for (uint32_t k0 = 0; k0 < n; k0 += 8u) {
    float t[8];
#pragma unroll
    for (int j = 0; j < 8; j++) t[j] = p[min(k0 + j, n - 1u) * stride];
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (k0 + j < n) s += t[j];
  }
  return s;
}

// ------------------------------------------------------------------------------------------------ LDS table copies
__device__ __forceinline__ void copy_words16(uint32_t* dst, const uint32_t* src, int nwords, int tid, int nthreads) {
  const uint4* s = (const uint4*)src;
  uint4* d = (uint4*)dst;
  for (int i = tid; i < nwords / 4; i += nthreads) d[i] = s[i];
}


// floor(a / b) for a < 4096 and 0 < b <= 64 in four instructions instead of the forty of an integer division (wave
// counts and rows of a chunk): (a + 0.5) / b lies at least 1 / 128 away from every integer, and the float product is
// within 1 / 1024 of it.
__device__ __forceinline__ uint32_t small_div(uint32_t a, uint32_t b) {
  return (uint32_t)(((float)a + 0.5f) * __builtin_amdgcn_rcpf((float)b));
}

// One piece of a workgroup's prologue copy into LDS: n16 16-byte items from device memory to the LDS word offset dst;
// pad_shift: 0, or four words of padding follow every 1 << pad_shift items (3: fp32 activations for the padded rows of
// XLds below, 2: fp16 activations in the same arrangement, see XHalf).
struct CopyJob {
  const uint4* src;
  uint32_t dst, n16;
  uint32_t pad_shift;
};
// All pieces as one pass over their concatenation, K items per thread in flight: every load of a batch is requested
// before the first LDS store waits for one (piece by piece, each copy would cost its own round trip to memory).
// Indices past the end repeat the last item (no branch around a load); only the stores are conditional.
template <int K, int NJ>
__device__ __forceinline__ void copy_jobs(uint32_t* smem, const CopyJob (&jobs)[NJ], uint32_t tid, uint32_t nt) {
  uint32_t total = 0;
#pragma unroll
  for (int j = 0; j < NJ; j++) total += jobs[j].n16;
  if (total == 0) return;
  for (uint32_t base = tid; base < total; base += K * nt) {
    uint4 v[K];
    uint32_t dw[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
      const uint32_t i = min(base + k * nt, total - 1u);
      // the piece item i falls in: the last one that starts at or before i (pieces of no items are passed over)
      const uint4* src = jobs[0].src;
      uint32_t dst = jobs[0].dst, ps = jobs[0].pad_shift, loc = i, first = 0;
#pragma unroll
      for (int j = 1; j < NJ; j++) {
        first += jobs[j - 1].n16;
        if (i >= first) { src = jobs[j].src; dst = jobs[j].dst; ps = jobs[j].pad_shift; loc = i - first; }
      }
      v[k] = src[loc];
      dw[k] = dst + 4u * loc + (ps ? (loc >> ps) * 4u : 0u);
    }
#pragma unroll
    for (int k = 0; k < K; k++)
      if (base + k * nt < total) *(uint4*)(smem + dw[k]) = v[k];
  }
}

// Waits until at most N of the wave's vector memory operations are outstanding, and keeps the compiler from moving memory
// accesses across the wait (s_waitcnt: the count's low four bits in bits 0-3, its high two in bits 14-15; the other
// counters at their maxima, i.e. not waited for). For loads whose destination is LDS, which the compiler does not track.
template <int N>
__device__ __forceinline__ void wait_vm() {
  static_assert(N >= 0 && N < 64, "s_waitcnt holds six bits of vmcnt");
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}
// A piece of a prologue copy by loads that write LDS themselves (no registers in between, so the requests can be issued
// ahead of everything else a kernel asks memory for and cost nothing until the data is needed): the whole groups of 64
// items of the piece, dealt over the waves; item `slot` of the LDS region comes from src[perm(slot)] (a wave's load
// writes 64 consecutive 16-byte slots, lane l the l-th; where the data is read in another order the source index is
// permuted instead). Returns the number of items covered; the caller copies the rest, waits (wait_vm) and synchronises.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
// The same load, hidden from the compiler: it follows the builtin's LDS writes and puts a wait for every outstanding
// load in front of each LDS read it cannot prove disjoint from them (a read of one half of a double buffer while the
// other half is being filled), which would expose a full trip to memory per stage. Lane l's 16 bytes from byte
// offset voff + soff of the descriptor land at dst + 16 l (dst wave-uniform). Callers wait with wait_vm and must not
// use the builtin forms of LDS-direct loads, movrel or other users of M0 in the same kernel: M0 is not restored.
__device__ __forceinline__ void lds_dma16(rsrc_t rs, const void* dst, uint32_t voff, uint32_t soff) {
  const uint32_t at = (uint32_t)(uintptr_t)(lds_ptr_t)dst;
  // (a scalar write of M0 wants one wait state before an instruction that reads it as the LDS address)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" : : "s"(at), "v"(voff), "s"(rs), "s"(soff) : "memory");
}
template <class PERM>
__device__ __forceinline__ uint32_t lds_dma_groups(uint32_t* dst, const uint4* src, uint32_t n16, uint32_t wave, uint32_t nwaves,
                                                   uint32_t lane, PERM perm) {
  // (the buffer form of the load: the compiler orders later LDS reads behind the global form with waits for every
  // outstanding load, which would serialise a kernel's weight-row pipeline; callers wait explicitly instead)
  const uint32_t groups = n16 >> 6;
  const rsrc_t rs = make_rsrc(src, n16 * 16u);
  for (uint32_t g = wave; g < groups; g += nwaves)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)(dst + 256u * g), 16, (int)(16u * perm(64u * g + lane)), 0, 0, 0);
  return groups << 6;
}

// table piece k of decoder D for copy_jobs (an empty piece when D stages no such table or is not in use)
template <class D>
__device__ __forceinline__ CopyJob tbl_job_of(int k, uint32_t at, bool live) {
  if constexpr (requires { D::NTBL; }) {
    if (live && k < D::NTBL) return D::tbl_job(k, at);
  }
  return {nullptr, 0u, 0u, 0u};
}

// ------------------------------------------------------------------------------------------------ x slices
// 32 consecutive activations -> 16 fp16 pairs (round to nearest even) + the sum of the rounded values
struct X32 {
  uint32_t v[16];
  float sx;
};
// Where load_x() finds the activations: plain memory (const float*), or a workgroup's LDS copy (XLds) in which every
// 32-float slice is followed by four floats of padding. A lane's slice of a row is 32 (or 8, or 16) consecutive
// floats, so read straight from device memory each 128-bit load of a wave touches 64 different cache lines; staged with
// contiguous loads and read back from the padded LDS rows (36 words apart: 16 consecutive lanes hit 16 different bank
// quads) the same data costs one pass over the row per workgroup. Runs handed to one vector load never cross a slice.
struct XLds { const float* p; };
__device__ __forceinline__ const float* xat(const float* x, uint32_t col) { return x + col; }
__device__ __forceinline__ const float* xat(XLds x, uint32_t col) { return x.p + col + (col >> 5) * 4u; }
__host__ __device__ constexpr uint32_t xlds_words(uint32_t cols) { return cols + (cols >> 5) * 4u; }
// Cooperative copy of the first G (<= GMAX, workgroup-uniform) activation rows src[g] of n floats each (multiple of
// 4) into consecutive padded LDS rows of roww words. Every thread has up to K 128-bit loads per row in flight, all
// rows requested before the first store waits. Indices past the end of a row repeat its last item (no branch around
// load); only the stores are conditional, so all GMAX pointers must be readable.
template <int GMAX, int K = 4>
__device__ __forceinline__ void stage_x_rows(float* dst, const float* const (&src)[GMAX], uint32_t G, uint32_t roww, uint32_t n,
                                             uint32_t tid, uint32_t nt) {
  const uint32_t n4 = n >> 2;
  for (uint32_t base = tid; base < n4; base += K * nt) {
    u32x4 v[GMAX][K];  // (a plain vector type: arrays of the HIP struct types can end up in scratch memory)
#pragma unroll
    for (int g = 0; g < GMAX; g++) {  // every src[g] is readable (rows past G are loaded and dropped)
#pragma unroll
      for (int k = 0; k < K; k++) v[g][k] = ((const u32x4*)src[g])[min(base + k * nt, n4 - 1u)];
    }
#pragma unroll
    for (int g = 0; g < GMAX; g++) {
      if (g < (int)G) {
#pragma unroll
        for (int k = 0; k < K; k++) {
          const uint32_t i = base + k * nt;
          if (i < n4) *(u32x4*)(dst + g * roww + 4u * i + (i >> 3) * 4u) = v[g][k];
        }
      }
    }
  }
}
// s: an exact power-of-two factor applied before the rounding to fp16 (callers undo it on their sums); it moves small
// activations out of the fp16 denormal range
__device__ __forceinline__ void load_x32_consecutive(const float* x, uint32_t* v, int n, float s = 1.f) {
  const float4* p = (const float4*)x;
#pragma unroll
  for (int i = 0; i < n / 4; i++) {
    const float4 f = p[i];
    v[2 * i] = pack_h2(f.x * s, f.y * s);
    v[2 * i + 1] = pack_h2(f.z * s, f.w * s);
  }
}
// sum of 2 n fp16 values in fp32: one dot product with (1, 1) per pair instead of two conversions and two additions
__device__ __forceinline__ float sum_h2(const uint32_t* v, int n) {
  const h2_t one = {(_Float16)1, (_Float16)1};
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < n; i++) s = __builtin_amdgcn_fdot2(as_h2(v[i]), one, s, false);
  return s;
}

// Activations that are already fp16 pairs (the h of the MoE layer, scaled and rounded by the kernel that wrote it): a
// 32-value slice is 16 words, read as it is. Staged in LDS, four words of padding follow every slice (20 words apart:
// 16 consecutive lanes hit 16 different bank quads, as with XLds).
__host__ __device__ constexpr uint32_t xhalf_words(uint32_t cols) { return (cols >> 5) * 20u; }
// The same slices without padding, for copies that cannot pad (loads that write LDS directly): slice u takes 16 words and
// its four 16-byte items are rotated by u / 2, item c at word 16 u + 4 ((c + (u >> 1)) & 3) -- sixteen consecutive lanes
// reading their item c then touch every group of four banks exactly twice, the least a 16-byte read of sixteen lanes can.
__device__ __forceinline__ uint32_t xhalf_rot_src(uint32_t slot) {  // the source item that belongs in 16-byte slot `slot`
  const uint32_t u = slot >> 2;
  return 4u * u + ((slot - (u >> 1)) & 3u);
}
__device__ __forceinline__ X32 load_x32_half(const uint32_t* p) {
  X32 r;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32x4 q = ((const u32x4*)p)[i];
    r.v[4 * i] = q.x; r.v[4 * i + 1] = q.y; r.v[4 * i + 2] = q.z; r.v[4 * i + 3] = q.w;
  }
  r.sx = sum_h2(r.v, 16);
  return r;
}
__device__ __forceinline__ X32 load_x32_half_rot(const uint32_t* region, uint32_t u) {  // slice u of a region in the rotated layout
  X32 r;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32x4 q = *(const u32x4*)(region + 16u * u + 4u * ((i + (u >> 1)) & 3u));
    r.v[4 * i] = q.x; r.v[4 * i + 1] = q.y; r.v[4 * i + 2] = q.z; r.v[4 * i + 3] = q.w;
  }
  r.sx = sum_h2(r.v, 16);
  return r;
}

// ================================================================================================ decoders (n = 1)
// Interface of a decoder D:
//   UNIT            columns one lane owns per unit
//   LDS_WORDS       32-bit words of table the workgroup stages in LDS (0 = none)
//   fill_lds()      cooperative table copy
//   STAGE_X         a lane's slice is one run of 128 bytes: read straight from device memory every 128-bit load of a
//                   wave touches 64 cache lines, so the workgroup stages the row in LDS with contiguous loads instead
//                   (decoders whose slices are runs of 32 or 64 bytes read them directly: 16 or 32 lines per load)
//   X / load_x()    the lane's activation slice for unit u of a row (x points at the row's first activation)
//   Raw / load()    the raw block bytes of unit u of a weight row (global loads only, so callers can prefetch)
//   dot()           sum over the unit's columns of weight * activation, fp32

// ---- IQ1_S: {fp16 d; u8 qs[32]; u16 qh[8]}, 50 bytes / 256 weights; unit = one 32-weight sub-block
struct DecIQ1S {
  static constexpr int UNIT = 32, GRID_WORDS = MSQ_IQ1S_GRID_N * 4, LDS_WORDS = GRID_WORDS + 32;
  static constexpr uint32_t BLOCK = 50, UPB = 8;  // bytes of a block, units in it
  static constexpr bool STAGE_X = true;
  typedef X32 X;
  struct Raw { uint32_t qs, qh, d; };
  // The two sub-block factors of a unit, {2 s + 1, delta (2 s + 1)}, come from the table behind the grid: one 8-byte read
  // (sixteen entries in distinct banks: conflict-free) instead of six vector instructions.
  __device__ static float2 factors(const Raw& r, const uint32_t* lds) {
    return *(const float2*)((const uint8_t*)lds + GRID_WORDS * 4 + ((r.qh >> 9) & 0x78u));
  }
  // d (2 s + 1) (acc + delta sx)
  __device__ static float scaled(const Raw& r, float2 f, float acc, float sx) {
    return half_bits_to_float(r.d) * __builtin_fmaf(f.x, acc, f.y * sx);
  }
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) { copy_words16(lds, g_tbl_iq1s.w, LDS_WORDS, tid, nt); }
  static constexpr int NTBL = 1;
  __device__ static CopyJob tbl_job(int, uint32_t at) { return {(const uint4*)g_tbl_iq1s.w, at, LDS_WORDS / 4, 0u}; }
  template <class S>
  __device__ static X load_x(S x, uint32_t u, float s = 1.f) {
    X r;
    load_x32_consecutive(xat(x, 32u * u), r.v, 32, s);
    r.sx = sum_h2(r.v, 16);
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    const P b = row + (u >> 3) * 50u;
    const uint32_t ib = u & 7u;
    return {ld32(b + 2 + 4 * ib), ld16(b + 34 + 2 * ib), ld16(b)};
  }
  // the same bytes through a buffer descriptor: Off holds the lane's byte offsets inside a row, soff the row's offset
  struct Off { uint32_t qs, qh, d; };
  static constexpr int FETCH_LOADS = 3;  // loads of one fetch()
  __device__ static Off offsets(uint32_t u) {
    const uint32_t b = (u >> 3) * 50u, ib = u & 7u;
    return {b + 2 + 4 * ib, b + 34 + 2 * ib, b};
  }
  __device__ static Raw fetch(rsrc_t rs, const Off& o, uint32_t soff) {
    return {buf_ld32(rs, o.qs, soff), buf_ld16(rs, o.qh, soff), buf_ld16(rs, o.d, soff)};
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t* lds) {
    const uint4* grid = (const uint4*)lds;
    float acc = 0.f;
#pragma unroll
    for (int l = 0; l < 4; l++) {
      const uint32_t idx = ((r.qs >> (8 * l)) & 0xFFu) | (((r.qh >> (3 * l)) & 7u) << 8);
      const uint4 g = grid[idx];
      acc = dot2(g.x, x.v[4 * l + 0], acc);
      acc = dot2(g.y, x.v[4 * l + 1], acc);
      acc = dot2(g.z, x.v[4 * l + 2], acc);
      acc = dot2(g.w, x.v[4 * l + 3], acc);
    }
    return scaled(r, factors(r, lds), acc, x.sx);
  }
  // the same dot split for software pipelining: lookup() only issues the table reads of a stage, partial() consumes
  // them (the last stage applies the scale), so a caller can keep the next stage's reads in flight during the math
  static constexpr int STAGES = 1;
  struct Look { uint4 g[4]; float2 f; };
  __device__ static Look lookup(const Raw& r, int, const uint32_t* lds) {
    const uint8_t* grid = (const uint8_t*)lds;
    Look k;
    k.f = factors(r, lds);
#pragma unroll
    for (int l = 0; l < 4; l++) {
      const uint32_t off = (((r.qs >> (8 * l)) & 0xFFu) << 4) | (((r.qh >> (3 * l)) & 7u) << 12);
      k.g[l] = *(const uint4*)(grid + off);
    }
    return k;
  }
  __device__ static float partial(const Raw& r, const Look& k, const X& x, int, float) {
    // two interleaved chains: a dependent dot2 issues every 8 cycles, an independent one every 4
    float acc = 0.f, acc1 = 0.f;
#pragma unroll
    for (int l = 0; l < 4; l += 2) {
      acc = dot2(k.g[l].x, x.v[4 * l + 0], acc);
      acc1 = dot2(k.g[l + 1].x, x.v[4 * l + 4], acc1);
      acc = dot2(k.g[l].y, x.v[4 * l + 1], acc);
      acc1 = dot2(k.g[l + 1].y, x.v[4 * l + 5], acc1);
      acc = dot2(k.g[l].z, x.v[4 * l + 2], acc);
      acc1 = dot2(k.g[l + 1].z, x.v[4 * l + 6], acc1);
      acc = dot2(k.g[l].w, x.v[4 * l + 3], acc);
      acc1 = dot2(k.g[l + 1].w, x.v[4 * l + 7], acc1);
    }
    acc += acc1;
    return scaled(r, k.f, acc, x.sx);
  }
};

// ---- IQ2_XXS: {fp16 d; u16 qs[32]}, 66 bytes / 256 weights; unit = one 32-weight sub-block (8 bytes)
struct DecIQ2XXS {
  static constexpr int UNIT = 32, LDS_WORDS = MSQ_IQ2XXS_GRID_N * 4 + 128 * 4;
  static constexpr uint32_t BLOCK = 66, UPB = 8;  // bytes of a block, units in it
  static constexpr bool STAGE_X = true;
  typedef X32 X;
  struct Raw { uint32_t a0, a1, d; };
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) {
    copy_words16(lds, g_tbl_iq2xxs.w, MSQ_IQ2XXS_GRID_N * 4, tid, nt);
    copy_words16(lds + MSQ_IQ2XXS_GRID_N * 4, g_tbl_sign.w, 128 * 4, tid, nt);
  }
  static constexpr int NTBL = 2;
  __device__ static CopyJob tbl_job(int k, uint32_t at) {
    if (k == 0) return {(const uint4*)g_tbl_iq2xxs.w, at, MSQ_IQ2XXS_GRID_N, 0u};
    return {(const uint4*)g_tbl_sign.w, at + MSQ_IQ2XXS_GRID_N * 4, 128, 0u};
  }
  template <class S>
  __device__ static X load_x(S x, uint32_t u, float s = 1.f) {
    X r;
    load_x32_consecutive(xat(x, 32u * u), r.v, 32, s);
    r.sx = 0.f;
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    const P b = row + (u >> 3) * 66u;
    const u64_a2 a = ld64(b + 2 + 8 * (u & 7u));
    return {a.x, a.y, ld16(b)};
  }
  struct Off { uint32_t a, d; };
  static constexpr int FETCH_LOADS = 2;  // loads of one fetch()
  __device__ static Off offsets(uint32_t u) {
    const uint32_t b = (u >> 3) * 66u;
    return {b + 2 + 8 * (u & 7u), b};
  }
  __device__ static Raw fetch(rsrc_t rs, const Off& o, uint32_t soff) {
    const u64_a2 a = buf_ld64(rs, o.a, soff);
    return {a.x, a.y, buf_ld16(rs, o.d, soff)};
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t* lds) {
    const uint4* grid = (const uint4*)lds;
    const uint4* sign = (const uint4*)(lds + MSQ_IQ2XXS_GRID_N * 4);
    float acc = 0.f;
#pragma unroll
    for (int l = 0; l < 4; l++) {
      const uint4 g = grid[(r.a0 >> (8 * l)) & 0xFFu];
      const uint4 s = sign[(r.a1 >> (7 * l)) & 127u];
      acc = dot2(g.x ^ s.x, x.v[4 * l + 0], acc);
      acc = dot2(g.y ^ s.y, x.v[4 * l + 1], acc);
      acc = dot2(g.z ^ s.z, x.v[4 * l + 2], acc);
      acc = dot2(g.w ^ s.w, x.v[4 * l + 3], acc);
    }
    const float db = half_bits_to_float(r.d) * (0.5f + (float)(r.a1 >> 28)) * 0.25f;
    return db * acc;
  }
  // two pipeline stages of two grid entries each (see DecIQ1S)
  static constexpr int STAGES = 2;
  struct Look { uint4 g[2], s[2]; };
  __device__ static Look lookup(const Raw& r, int stage, const uint32_t* lds) {
    const uint8_t* grid = (const uint8_t*)lds;
    const uint8_t* sign = (const uint8_t*)(lds + MSQ_IQ2XXS_GRID_N * 4);
    Look k;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int l = 2 * stage + i;
      k.g[i] = *(const uint4*)(grid + (((r.a0 >> (8 * l)) & 0xFFu) << 4));
      k.s[i] = *(const uint4*)(sign + (((r.a1 >> (7 * l)) & 127u) << 4));
    }
    return k;
  }
  __device__ static float partial(const Raw& r, const Look& k, const X& x, int stage, float acc) {
    float acc1 = 0.f;  // second chain: dependent dot2s issue at half rate
    {
      const int l = 2 * stage;
      acc = dot2(k.g[0].x ^ k.s[0].x, x.v[4 * l + 0], acc);
      acc1 = dot2(k.g[1].x ^ k.s[1].x, x.v[4 * l + 4], acc1);
      acc = dot2(k.g[0].y ^ k.s[0].y, x.v[4 * l + 1], acc);
      acc1 = dot2(k.g[1].y ^ k.s[1].y, x.v[4 * l + 5], acc1);
      acc = dot2(k.g[0].z ^ k.s[0].z, x.v[4 * l + 2], acc);
      acc1 = dot2(k.g[1].z ^ k.s[1].z, x.v[4 * l + 6], acc1);
      acc = dot2(k.g[0].w ^ k.s[0].w, x.v[4 * l + 3], acc);
      acc1 = dot2(k.g[1].w ^ k.s[1].w, x.v[4 * l + 7], acc1);
    }
    acc += acc1;
    if (stage == 1) acc *= half_bits_to_float(r.d) * (0.5f + (float)(r.a1 >> 28)) * 0.25f;
    return acc;
  }
};

// ---- Q8_0: {fp16 d; int8 qs[32]}, 34 bytes / 32 weights; unit = one block, activations kept in fp32
struct DecQ8_0 {
  static constexpr int UNIT = 32, LDS_WORDS = 0;
  static constexpr uint32_t BLOCK = 34, UPB = 1;  // bytes of a block, units in it
  static constexpr bool STAGE_X = true;
  struct X { float v[32]; };
  struct Raw { uint32_t q[8]; uint32_t d; };
  __device__ static void fill_lds(uint32_t*, int, int) {}
  template <class S>
  __device__ static X load_x(S x, uint32_t u, float s = 1.f) {
    X r;
    const float4* p = (const float4*)xat(x, 32u * u);
#pragma unroll
    for (int i = 0; i < 8; i++) { const float4 f = p[i]; r.v[4 * i] = f.x * s; r.v[4 * i + 1] = f.y * s; r.v[4 * i + 2] = f.z * s; r.v[4 * i + 3] = f.w * s; }
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    const P b = row + u * 34u;
    const u128_a2 a = ld128(b + 2), c = ld128(b + 18);
    return {{a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w}, ld16(b)};
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t*) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t q = r.q[i];
      acc += (float)(int8_t)(q & 0xFF) * x.v[4 * i];
      acc += (float)(int8_t)((q >> 8) & 0xFF) * x.v[4 * i + 1];
      acc += (float)(int8_t)((q >> 16) & 0xFF) * x.v[4 * i + 2];
      acc += (float)(int8_t)(q >> 24) * x.v[4 * i + 3];
    }
    return half_bits_to_float(r.d) * acc;
  }
};

// ---- IQ4_NL: {fp16 d; u8 qs[16]}, 18 bytes / 32 weights; byte j holds columns j (low nibble) and j + 16 (high)
struct DecIQ4NL {
  static constexpr int UNIT = 32, LDS_WORDS = 256;
  static constexpr uint32_t BLOCK = 18, UPB = 1;  // bytes of a block, units in it
  static constexpr bool STAGE_X = true;
  struct X { uint32_t v[16]; };  // pair j = (x[j], x[j + 16])
  struct Raw { uint32_t q[4]; uint32_t d; };
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) { copy_words16(lds, g_tbl_iq4nl.w, 256, tid, nt); }
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    X r;
    const float4* p = (const float4*)xat(x, 32u * u);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float4 a = p[i], b = p[i + 4];
      r.v[4 * i] = pack_h2(a.x, b.x); r.v[4 * i + 1] = pack_h2(a.y, b.y);
      r.v[4 * i + 2] = pack_h2(a.z, b.z); r.v[4 * i + 3] = pack_h2(a.w, b.w);
    }
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    const P b = row + u * 18u;
    const u128_a2 a = ld128(b + 2);
    return {{a.x, a.y, a.z, a.w}, ld16(b)};
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t* lds) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int k = 0; k < 4; k++) acc = dot2(lds[(r.q[i] >> (8 * k)) & 0xFFu], x.v[4 * i + k], acc);
    }
    return half_bits_to_float(r.d) * acc;
  }
};

// ---- Q6_K: {u8 ql[128]; u8 qh[64]; int8 sc[16]; fp16 d}, 210 bytes / 256 weights.
// Unit j of a block (8 per block): half h = j >> 2, l0 = 8 * (j & 3); it owns the four 8-column runs
// 128 h + 32 k + l0 .. + 7 (k = 0..3), which share the bytes ql[64 h + l0 ..], ql[64 h + 32 + l0 ..], qh[32 h + l0 ..].
struct DecQ6K {
  static constexpr int UNIT = 32, LDS_WORDS = 0;
  static constexpr uint32_t BLOCK = 210, UPB = 8;  // bytes of a block, units in it
  static constexpr bool STAGE_X = false;
  struct X { uint32_t v[16]; float sx[4]; };
  struct Raw { uint32_t qa[2], qb[2], qh[2], sc[2], d; };
  __device__ static void fill_lds(uint32_t*, int, int) {}
  template <class S>
  __device__ static X load_x(S x, uint32_t u, float s = 1.f) {
    X r;
    const uint32_t j = u & 7u;
    const uint32_t base = 256u * (u >> 3) + 128u * (j >> 2) + 8u * (j & 3u);
#pragma unroll
    for (int k = 0; k < 4; k++) {
      load_x32_consecutive(xat(x, base + 32u * k), r.v + 4 * k, 8, s);
      r.sx[k] = sum_h2(r.v + 4 * k, 4);
    }
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    const P b = row + (u >> 3) * 210u;
    const uint32_t j = u & 7u, h = j >> 2, l0 = 8u * (j & 3u);
    const u64_a2 a = ld64(b + 64 * h + l0), c = ld64(b + 64 * h + 32 + l0), q = ld64(b + 128 + 32 * h + l0);
    const u64_a2 s = ld64(b + 192 + 8 * h);
    return {{a.x, a.y}, {c.x, c.y}, {q.x, q.y}, {s.x, s.y}, ld16(b + 208)};
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t*, uint32_t u) {
    const uint32_t is = (u >> 1) & 1u;  // l0 / 16
    const float d = half_bits_to_float(r.d);
    float total = 0.f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
      float acc = 0.f;
#pragma unroll
      for (int w = 0; w < 2; w++) {
        const uint32_t src = (k & 1) ? r.qb[w] : r.qa[w];
        const uint32_t n = (src >> (4 * (k >> 1))) & 0x0F0F0F0Fu;
        const uint32_t hb = ((r.qh[w] >> (2 * k)) & 0x03030303u) << 4;
        const uint32_t q = n | hb;  // 4 bytes in 0..63
        acc = dot2(bytes01_to_h2_1024(q), x.v[4 * k + 2 * w], acc);
        acc = dot2(bytes23_to_h2_1024(q), x.v[4 * k + 2 * w + 1], acc);
      }
      // scale byte index 2k + is lies in word k >> 1
      const int sc = (int)(int8_t)((r.sc[k >> 1] >> (8u * ((2u * k & 3u) + is))) & 0xFFu);
      total += d * (float)sc * (acc - 1056.f * x.sx[k]);  // halves carry 1024 + q6; weight = q6 - 32
    }
    return total;
  }
};

// ---- Q5_K: {fp16 d, dmin; u8 sc[12]; u8 qh[32]; u8 ql[128]}, 176 bytes / 256 weights.
// Unit j of a block: 64-column group g = j >> 1, l0 = 16 * (j & 1); it owns columns 64 g + l0 .. + 15 (low nibbles,
// scale index 2 g) and 64 g + 32 + l0 .. + 15 (high nibbles, scale index 2 g + 1).
struct DecQ5K {
  static constexpr int UNIT = 32, LDS_WORDS = 0;
  static constexpr uint32_t BLOCK = 176, UPB = 8;  // bytes of a block, units in it
  static constexpr bool STAGE_X = false;
  struct X { uint32_t v[16]; float sx[2]; };
  struct Raw { uint32_t ql[4], qh[4], pa, pb, pc, dd; };
  __device__ static void fill_lds(uint32_t*, int, int) {}
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    X r;
    const uint32_t j = u & 7u;
    const uint32_t base = 256u * (u >> 3) + 64u * (j >> 1) + 16u * (j & 1u);
    load_x32_consecutive(xat(x, base), r.v, 16);
    load_x32_consecutive(xat(x, base + 32u), r.v + 8, 16);
    r.sx[0] = sum_h2(r.v, 8);
    r.sx[1] = sum_h2(r.v + 8, 8);
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    const P b = row + (u >> 3) * 176u;
    const uint32_t j = u & 7u, g = j >> 1, l0 = 16u * (j & 1u), is = 2u * g;
    const u128_a2 l = ld128(b + 48 + 32 * g + l0), h = ld128(b + 16 + l0);
    // scale bytes is, is+1 (pa), is+4, is+5 (pb) and, for the upper groups, is-4, is-3 (pc)
    return {{l.x, l.y, l.z, l.w}, {h.x, h.y, h.z, h.w}, ld16(b + 4 + is), ld16(b + 8 + is),
            ld16(b + (is >= 4 ? is : 4u)), ld32(b)};
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t*, uint32_t u) {
    const uint32_t g = (u & 7u) >> 1;
    const float d = half_bits_to_float(r.dd & 0xFFFFu), dmin = half_bits_to_float(r.dd >> 16);
    float total = 0.f;
#pragma unroll
    for (int run = 0; run < 2; run++) {
      float acc = 0.f;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        const uint32_t n = (r.ql[w] >> (4 * run)) & 0x0F0F0F0Fu;
        const uint32_t hb = ((r.qh[w] >> (2 * g + run)) & 0x01010101u) << 4;
        const uint32_t q = n | hb;  // 4 bytes in 0..31
        acc = dot2(bytes01_to_h2_1024(q), x.v[8 * run + 2 * w], acc);
        acc = dot2(bytes23_to_h2_1024(q), x.v[8 * run + 2 * w + 1], acc);
      }
      const uint32_t a = (r.pa >> (8 * run)) & 0xFFu, bq = (r.pb >> (8 * run)) & 0xFFu, c = (r.pc >> (8 * run)) & 0xFFu;
      uint32_t sc, mn;
      if (g < 2) { sc = a & 63u; mn = bq & 63u; }
      else { sc = (bq & 0xFu) | ((c >> 6) << 4); mn = (bq >> 4) | ((a >> 6) << 4); }
      total += (d * (float)sc) * (acc - 1024.f * x.sx[run]) - (dmin * (float)mn) * x.sx[run];
    }
    return total;
  }
};

// ---- dense rows (F32 / F16 / BF16): unit = 8 consecutive elements, fp32 activations
template <int QT>
struct DecDense {
  static constexpr int UNIT = 8, LDS_WORDS = 0;
  static constexpr bool STAGE_X = false;
  struct X { float v[8]; };
  struct Raw { uint32_t w[QT == MSQ_F32 ? 8 : 4]; };
  __device__ static void fill_lds(uint32_t*, int, int) {}
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    X r;
    const float4* p = (const float4*)xat(x, 8u * u);
    const float4 a = p[0], b = p[1];
    r.v[0] = a.x; r.v[1] = a.y; r.v[2] = a.z; r.v[3] = a.w; r.v[4] = b.x; r.v[5] = b.y; r.v[6] = b.z; r.v[7] = b.w;
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    Raw r;
    if constexpr (QT == MSQ_F32) {
      const u128_a2 a = ld128(row + 32u * u), b = ld128(row + 32u * u + 16);
      r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w; r.w[4] = b.x; r.w[5] = b.y; r.w[6] = b.z; r.w[7] = b.w;
    } else {
      const u128_a2 a = ld128(row + 16u * u);
      r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w;
    }
    return r;
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t*) {
    float acc = 0.f;
    if constexpr (QT == MSQ_F32) {
#pragma unroll
      for (int i = 0; i < 8; i++) acc += __builtin_bit_cast(float, r.w[i]) * x.v[i];
    } else if constexpr (QT == MSQ_F16) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        acc += half_bits_to_float(r.w[i] & 0xFFFFu) * x.v[2 * i];
        acc += half_bits_to_float(r.w[i] >> 16) * x.v[2 * i + 1];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        acc += __builtin_bit_cast(float, r.w[i] << 16) * x.v[2 * i];
        acc += __builtin_bit_cast(float, r.w[i] & 0xFFFF0000u) * x.v[2 * i + 1];
      }
    }
    return acc;
  }
};

// Uniform call: decoders whose dot() needs the unit index (sub-position inside the block) take it as 4th argument.
template <class D>
__device__ __forceinline__ float dec_dot(const typename D::Raw& r, const typename D::X& x, const uint32_t* lds, uint32_t u) {
  if constexpr (requires { D::dot(r, x, lds, u); }) return D::dot(r, x, lds, u);
  else return D::dot(r, x, lds);
}

}  // namespace msq
