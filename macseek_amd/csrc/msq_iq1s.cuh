// IQ1_S decoder for the one-token MoE kernels: integer dot products over 16-bit block-fixed-point activations.
//
// Block layout {fp16 d; u8 qs[32]; u16 qh[8]} and the arithmetic w = d * (2 s + 1) * (grid + delta), delta = -+ 1/8,
// follow the reference's CPU dequantizer (tests/ref/dequant.cpp:77-91). What is this library's own:
//   * a 32-weight unit is four grid entries of eight trits. The table holds 8 * (grid + delta) = 8 g +- 1 as int8, one
//     variant per sign of delta, so a unit's dot product is 16 v_dot4_i32_i8 against activations split into a low and a
//     high signed byte plane and nothing else depends on delta;
//   * activations are quantized per unit (32 columns): x ~ xs * n with |n| <= 32639 an integer and xs a power of two
//     times a constant, so a unit's integer sum is exact (|sum| < 2^24) and the rounding of an activation is 2^-16 of
//     its unit's largest value (about six times finer than rounding to fp16);
//   * every lookup address is assembled from whole bytes. Entry (b = qs byte, h = 3 bits of qh, sign of delta) lives at
//     LDS byte (b << 8) | (c << 7) | (sign << 6) | (h << 3), c = lane & 1 (two copies: with the 256-byte pitch that
//     byte-aligning b costs, one copy would sit in half of the banks). Two 256-entry tables indexed by the bytes of qh
//     hold the low address bytes of the four lookups already in place (and the sub-block scale 2 s + 1), so the four
//     addresses cost one v_or3 and four v_perm; a table read costs the CU about as much as five vector instructions
//     cost a SIMD, which is why there are two of them and not more.
#pragma once
#include "msq_device.cuh"

namespace msq {

// ------------------------------------------------------------------------------------------------ constant tables
// Image of one LDS copy without its gaps: 8-byte item ((b * 2 + sign) * 8 + h) holds the eight int8 values 8 g + 1
// (sign 0: delta = +1/8) or 8 g - 1 (sign 1) of grid entry (h << 8) | b.
struct TblIQ1S8 { uint32_t w[MSQ_IQ1S_GRID_N * 2 * 2]; };

constexpr TblIQ1S8 make_iq1s8() {
  TblIQ1S8 t{};
  for (int i = 0; i < MSQ_IQ1S_GRID_N; i++) {
    const int h = i >> 8, b = i & 255;
    for (int sign = 0; sign < 2; sign++) {
      unsigned c = msq_iq1s_code[i];
      const int at = 2 * ((b * 2 + sign) * 8 + h);
      for (int j = 0; j < 8; j++, c /= 3) {
        const int v = 8 * ((int)(c % 3) - 1) + (sign ? -1 : 1);
        t.w[at + j / 4] |= (uint32_t)(uint8_t)(int8_t)v << (8 * (j % 4));
      }
    }
  }
  return t;
}
__device__ __attribute__((aligned(16))) const TblIQ1S8 g_tbl_iq1s8 = make_iq1s8();

// ------------------------------------------------------------------------------------------------ quantized activations
// One unit = 32 consecutive activations, stored as 20 words: 8 words of low bytes, 8 words of high bytes (column j of
// the unit in byte j of its plane), an eighth of the scale xs as a float, three words of padding (consecutive units are
// 80 bytes apart: sixteen lanes reading 16 bytes each hit sixteen different bank quads).
constexpr uint32_t kXqWords = 20;
__host__ __device__ constexpr uint32_t xq_words(uint32_t cols) { return cols / 32u * kXqWords; }
struct XQLds { const uint32_t* p; };

// x = xs * n: n = round(x * 2^-e * (1 - 2^-8) * 32767) with 2^e the power of two above the unit's largest |x|, so
// |n| <= 32639 and n + 128 still fits 16 bits; split n = 256 * nh + nl with both bytes signed.
constexpr float kXqShrink = 0.99609375f;                         // 1 - 2^-8
constexpr float kXqUnit = 1.0f / (32767.0f * 0.99609375f);      // xs = kXqUnit * 2^e
__device__ __forceinline__ int xq_exponent(float m) { return (int)((__builtin_bit_cast(uint32_t, m) >> 23) & 0xFFu) - 126; }
typedef short s2_t __attribute__((ext_vector_type(2)));
typedef unsigned short us2_t __attribute__((ext_vector_type(2)));
// four activations -> their low-byte word and high-byte word
__device__ __forceinline__ void xq_quant4(float4 v, float mult, uint32_t& lo, uint32_t& hi) {
  const s2_t p0 = __builtin_amdgcn_cvt_pknorm_i16(v.x * mult, v.y * mult), p1 = __builtin_amdgcn_cvt_pknorm_i16(v.z * mult, v.w * mult);
  const us2_t r = {128, 128};
  const uint32_t q0 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(us2_t, p0) + r);
  const uint32_t q1 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(us2_t, p1) + r);
  lo = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, p1), __builtin_bit_cast(uint32_t, p0), 0x06040200u);
  hi = __builtin_amdgcn_perm(q1, q0, 0x07050301u);
}
// first product of a v_dot4_i32_i8 chain: the three-operand form with a literal zero addend (the compiler's choice, the
// two-operand accumulate form, needs an instruction to clear its accumulator first)
__device__ __forceinline__ int sdot4z(uint32_t a, uint32_t b) {
  int r;
  asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
template <int CTRL>
__device__ __forceinline__ float dpp_maxf(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
  return fmaxf(v, __builtin_bit_cast(float, moved));
}
// Cooperative form: the workgroup quantizes n floats (a multiple of 32; 16-byte aligned) into n / 32 units at dst.
// Thread t takes the float4 items t, t + nt, ...; the eight lanes that share a unit agree on its largest value
// through three DPP exchanges. A batch of K items per thread is requested (xq_issue) before it is quantized and
// stored (xq_finish), so a caller can put its other loads in flight in between.
template <int K>
struct XqBatch { f4_t v[K]; };  // (plain vector types: arrays of the HIP struct types can end up in scratch memory)
template <int K>
__device__ __forceinline__ XqBatch<K> xq_issue(const float* src, uint32_t n4, uint32_t base, uint32_t nt) {
  XqBatch<K> b;
#pragma unroll
  for (int k = 0; k < K; k++) b.v[k] = ((const f4_t*)src)[min(base + k * nt, n4 - 1u)];
  return b;
}
template <int K>
__device__ __forceinline__ void xq_finish(uint32_t* dst, const XqBatch<K>& b, uint32_t n4, uint32_t base, uint32_t nt) {
#pragma unroll
  for (int k = 0; k < K; k++) {
    const uint32_t i = base + k * nt;  // groups of eight lanes are in range, or out of it, together (n4 % 8 == 0)
    const float4 v = {b.v[k].x, b.v[k].y, b.v[k].z, b.v[k].w};
    float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    m = dpp_maxf<0x141>(m); m = dpp_maxf<0xB1>(m); m = dpp_maxf<0x4E>(m);
    const int e = xq_exponent(m);
    uint32_t lo, hi;
    xq_quant4(v, __builtin_ldexpf(kXqShrink, -e), lo, hi);
    if (i < n4) {
      uint32_t* u = dst + (i >> 3) * kXqWords;
      u[i & 7u] = lo;
      u[8u + (i & 7u)] = hi;
      if ((i & 7u) == 0) u[16] = __builtin_bit_cast(uint32_t, __builtin_ldexpf(kXqUnit, e - 3));
    }
  }
}
// whole rows: the first batch may have been issued by the caller already (first != nullptr)
template <int K>
__device__ __forceinline__ void stage_xq(uint32_t* dst, const float* src, uint32_t n, uint32_t tid, uint32_t nt,
                                         const XqBatch<K>* first = nullptr) {
  const uint32_t n4 = n >> 2;
  for (uint32_t base = tid; base < n4; base += K * nt) {
    if (first && base == tid) { xq_finish<K>(dst, *first, n4, base, nt); continue; }
    const XqBatch<K> b = xq_issue<K>(src, n4, base, nt);
    xq_finish<K>(dst, b, n4, base, nt);
  }
}

// ================================================================================================ decoder
struct DecIQ1SQ {
  static constexpr int UNIT = 32;
  // words: [0, 512) table of the high qh byte {address bytes, 2 s + 1 as a float}, [512, 768) table of the low qh
  // byte, then the two grid copies (the small tables come first so that every table base fits the 16-bit offset field
  // of a DS instruction)
  static constexpr int LUT_HI_AT = 0, LUT_LO_AT = 512, GRID_AT = 768, GRID_WORDS = 16384;
  static constexpr int LDS_WORDS = GRID_AT + GRID_WORDS;
  static constexpr bool STAGE_X = true, QUANT_X = true, HAS_PRE = true;
  static constexpr int STAGES = 1;
  struct X { uint32_t lo[8], hi[8]; float xs8; };
  // qh and d are held as halves (bit containers): a 16-bit integer would be zero-extended, by an extra instruction,
  // before each use, and their users read bytes / the low half only
  struct Raw { uint32_t qs; _Float16 qh, d; };

  // ---- tables. The grid comes from device memory (32 KB, two entries per 16-byte item; issue_tables requests a
  // thread's items, finish_tables writes each into both copies); the two small tables are computed.
  static constexpr uint32_t ITEMS = MSQ_IQ1S_GRID_N;  // 16-byte items of the image
  struct TblRegs { u32x4 v[2]; };
  __device__ static TblRegs issue_tables(uint32_t tid, uint32_t nt) {
    TblRegs r;
#pragma unroll
    for (int j = 0; j < 2; j++) r.v[j] = ((const u32x4*)g_tbl_iq1s8.w)[min(tid + j * nt, ITEMS - 1u)];
    return r;
  }
  __device__ static void finish_tables(uint32_t* lds, const TblRegs& r, uint32_t tid, uint32_t nt) {
    for (uint32_t b = tid; b < 256u; b += nt) {
      // high byte of qh: bit 0 = top bit of h2, bits 1..3 = h3, bits 4..6 = s, bit 7 = sign of delta (into every byte)
      const uint32_t sign = (b >> 7) * 0x40404040u;
      lds[LUT_HI_AT + 2 * b] = sign | ((b & 1u) << 21) | (((b >> 1) & 7u) << 27);
      lds[LUT_HI_AT + 2 * b + 1] = __builtin_bit_cast(uint32_t, (float)(2u * ((b >> 4) & 7u) + 1u));
      // low byte of qh: bits 0..2 = h0, bits 3..5 = h1, bits 6..7 = low bits of h2
      lds[LUT_LO_AT + b] = ((b & 7u) << 3) | (((b >> 3) & 7u) << 11) | (((b >> 6) & 3u) << 19);
    }
    // image byte o = 16 i = (b << 7) | (sign << 6) | (h << 3) goes to LDS byte (b << 8) | (c << 7) | (o & 127)
    auto put = [&](uint32_t i, const u32x4& v) {
      const uint32_t o = 16u * i, at = (((o & ~127u) << 1) | (o & 127u)) >> 2;
      *(u32x4*)(lds + GRID_AT + at) = v;
      *(u32x4*)(lds + GRID_AT + at + 32u) = v;
    };
#pragma unroll
    for (int j = 0; j < 2; j++)
      if (tid + j * nt < ITEMS) put(tid + j * nt, r.v[j]);
    if (2u * nt < ITEMS) {  // workgroups of fewer than 1024 threads fetch the rest here
      // (the index is recomputed behind a barrier the compiler cannot look through: hoisted to the kernel's start, this
      // loop's addresses cost every thread of the usual 1024-thread launch five spilled registers -- 4 MB of scratch
      // writes per launch)
      uint32_t t2 = tid;
      asm volatile("" : "+v"(t2));
      for (uint32_t i0 = t2 + 2u * nt; i0 < ITEMS; i0 += nt) put(i0, ((const u32x4*)g_tbl_iq1s8.w)[i0]);
    }
  }
  __device__ static void fill_lds(uint32_t* lds, uint32_t tid, uint32_t nt) { finish_tables(lds, issue_tables(tid, nt), tid, nt); }

  // ---- activations
  __device__ static X load_x(XQLds x, uint32_t u) {
    const uint4* p = (const uint4*)(x.p + u * kXqWords);
    const uint4 a = p[0], b = p[1], c = p[2], d = p[3];
    return {{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w}, {c.x, c.y, c.z, c.w, d.x, d.y, d.z, d.w},
            __builtin_bit_cast(float, x.p[u * kXqWords + 16])};
  }
  // the same quantization by one lane on its own (rows too long to stage; S: plain memory or the padded LDS rows of XLds)
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    const float4* p = (const float4*)xat(x, 32u * u);
    float4 v[8];
    float m = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      v[i] = p[i];
      m = fmaxf(m, fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w))));
    }
    const int e = xq_exponent(m);
    const float mult = __builtin_ldexpf(kXqShrink, -e);
    X r;
#pragma unroll
    for (int i = 0; i < 8; i++) xq_quant4(v[i], mult, r.lo[i], r.hi[i]);
    r.xs8 = __builtin_ldexpf(kXqUnit, e - 3);
    return r;
  }

  // ---- block bytes
  struct Off { uint32_t qs, qh, d; };
  __device__ static Off offsets(uint32_t u) {
    const uint32_t b = (u >> 3) * 50u, ib = u & 7u;
    return {b + 2 + 4 * ib, b + 34 + 2 * ib, b};
  }
  __device__ static Raw fetch(rsrc_t rs, const Off& o, uint32_t soff) {
    return {buf_ld32(rs, o.qs, soff), __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(rs, (int)o.qh, (int)soff, 0)),
            __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(rs, (int)o.d, (int)soff, 0))};
  }

  // ---- three-step decode: pre() reads the two qh tables, lookup() turns them into the four entry addresses and
  // reads the entries, partial() does the arithmetic. Each step of a unit is issued one unit ahead of the next.
  struct Pre { uint2 hi; uint32_t lo; };  // hi.x, lo: address bytes; hi.y: 2 s + 1
  struct Look { uint2 g[4]; float sc; };
  __device__ static Pre pre(const Raw& r, const uint32_t* lds) {
    const uint8_t* t = (const uint8_t*)lds;
    // byte selects read qh's two bytes directly (one instruction each; the bits above them never matter)
    uint32_t ahi, alo;
    asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(ahi) : "s"(3u), "v"(r.qh));
    asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(alo) : "s"(2u), "v"(r.qh));
    return {*(const uint2*)(t + LUT_HI_AT * 4 + ahi), *(const uint32_t*)(t + LUT_LO_AT * 4 + alo)};
  }
  // lanec: (lane & 1) * 0x80808080, the lane's grid copy in every byte
  __device__ static void lookup(const Raw& r, const Pre& a, const uint32_t* lds, uint32_t lanec, Look& k) {
    const uint8_t* t = (const uint8_t*)lds;
    const uint32_t T = a.hi.x | a.lo | lanec;
    k.g[0] = *(const uint2*)(t + GRID_AT * 4 + __builtin_amdgcn_perm(r.qs, T, 0x0c0c0400u));
    k.g[1] = *(const uint2*)(t + GRID_AT * 4 + __builtin_amdgcn_perm(r.qs, T, 0x0c0c0501u));
    k.g[2] = *(const uint2*)(t + GRID_AT * 4 + __builtin_amdgcn_perm(r.qs, T, 0x0c0c0602u));
    k.g[3] = *(const uint2*)(t + GRID_AT * 4 + __builtin_amdgcn_perm(r.qs, T, 0x0c0c0703u));
    k.sc = __builtin_bit_cast(float, a.hi.y);
  }
  __device__ static float partial(const Raw& r, const Look& k, const X& x) {
    // the first product of each chain takes a literal zero addend (three-operand form): no accumulator to clear
    int lo, hi;
    {
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(lo) : "v"(k.g[0].x), "v"(x.lo[0]));
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(hi) : "v"(k.g[0].x), "v"(x.hi[0]));
    lo = __builtin_amdgcn_sdot4((int)k.g[0].y, (int)x.lo[1], lo, false);
    hi = __builtin_amdgcn_sdot4((int)k.g[0].y, (int)x.hi[1], hi, false);
#pragma unroll
    for (int l = 1; l < 4; l++) {
      lo = __builtin_amdgcn_sdot4((int)k.g[l].x, (int)x.lo[2 * l], lo, false);
      hi = __builtin_amdgcn_sdot4((int)k.g[l].x, (int)x.hi[2 * l], hi, false);
      lo = __builtin_amdgcn_sdot4((int)k.g[l].y, (int)x.lo[2 * l + 1], lo, false);
      hi = __builtin_amdgcn_sdot4((int)k.g[l].y, (int)x.hi[2 * l + 1], hi, false);
    }
    }
    return finish(r, k, x, lo, hi);
  }
  __device__ static float finish(const Raw& r, const Look& k, const X& x, int lo, int hi) {
    const float t = (float)((hi << 8) + lo);  // sum of (8 g +- 1) * n over the unit, exact
    const float w = (t * x.xs8) * k.sc;
    float y;  // d * w with the fp16 d converted inside the multiply
    asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(y) : "v"(r.d), "v"(w));
    return y;
  }
  // two units against the same activations (gate and up of a row), their four chains interleaved: a wave on its own
  // issues a dependent product only every other slot
  __device__ static void partial2(const Raw& ra, const Look& ka, const Raw& rb, const Look& kb, const X& x, float& ya, float& yb) {
    int la, ha, lb, hb;
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(la) : "v"(ka.g[0].x), "v"(x.lo[0]));
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(ha) : "v"(ka.g[0].x), "v"(x.hi[0]));
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(lb) : "v"(kb.g[0].x), "v"(x.lo[0]));
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(hb) : "v"(kb.g[0].x), "v"(x.hi[0]));
    la = __builtin_amdgcn_sdot4((int)ka.g[0].y, (int)x.lo[1], la, false);
    ha = __builtin_amdgcn_sdot4((int)ka.g[0].y, (int)x.hi[1], ha, false);
    lb = __builtin_amdgcn_sdot4((int)kb.g[0].y, (int)x.lo[1], lb, false);
    hb = __builtin_amdgcn_sdot4((int)kb.g[0].y, (int)x.hi[1], hb, false);
#pragma unroll
    for (int l = 1; l < 4; l++) {
      la = __builtin_amdgcn_sdot4((int)ka.g[l].x, (int)x.lo[2 * l], la, false);
      ha = __builtin_amdgcn_sdot4((int)ka.g[l].x, (int)x.hi[2 * l], ha, false);
      lb = __builtin_amdgcn_sdot4((int)kb.g[l].x, (int)x.lo[2 * l], lb, false);
      hb = __builtin_amdgcn_sdot4((int)kb.g[l].x, (int)x.hi[2 * l], hb, false);
      la = __builtin_amdgcn_sdot4((int)ka.g[l].y, (int)x.lo[2 * l + 1], la, false);
      ha = __builtin_amdgcn_sdot4((int)ka.g[l].y, (int)x.hi[2 * l + 1], ha, false);
      lb = __builtin_amdgcn_sdot4((int)kb.g[l].y, (int)x.lo[2 * l + 1], lb, false);
      hb = __builtin_amdgcn_sdot4((int)kb.g[l].y, (int)x.hi[2 * l + 1], hb, false);
    }
    ya = finish(ra, ka, x, la, ha);
    yb = finish(rb, kb, x, lb, hb);
  }
};

}  // namespace msq
