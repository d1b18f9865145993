// Q6_K decoder for the gate/up kernel of the one-token MoE layer (the reference's shared-expert type): integer dot
// products over the 16-bit block-fixed-point activations of msq_iq1s.cuh. The fp16 decoder DecQ6K rounds x to 11
// significant bits, and on a shared expert (weight 1) that rounding is most of the layer's error against an
// F32-activation reference; here x is rounded at 2^-16 of the largest value of its 32 columns.
//
// Block layout {u8 ql[128]; u8 qh[64]; int8 sc[16]; fp16 d} and the arithmetic w = d sc (q - 32), q = low nibble |
// two high bits << 4, follow the reference's CPU dequantizer (tests/ref/dequant.cpp:60-76). The lane / unit mapping is
// DecQ6K's: unit j of a block owns four runs of eight columns, 128 (j >> 2) + 8 (j & 3) + 32 k for k = 0..3, so that it
// uses every bit of the bytes it loads; run k has its own int8 scale sc[8 (j >> 2) + 2 k + (j & 3) / 2] and lies in its
// own 32-column unit of the quantized activations (its own power-of-two scale xs_k). Per run: eight bytes q in 0..63
// against the low and the high byte plane of the activations (four v_dot4_i32_i8), and
//   sum w x = d sc xs_k (sum q n - 32 sum n),   n = 256 nh + nl the activation's integer,
// with 32 sum n precomputed per lane.
#pragma once
#include "msq_iq1s.cuh"

namespace msq {

struct DecQ6KQ {
  static constexpr int UNIT = 32, LDS_WORDS = 0;
  static constexpr uint32_t BLOCK = 210, UPB = 8;
  static constexpr bool STAGE_X = false, QUANT_X = true;  // (STAGE_X: the decode matvec reads its short runs directly, as DecQ6K)
  // per run k: two words of low bytes, two of high bytes, the scale, and -32 * sum n
  struct X { uint32_t lo[8], hi[8]; float xs[4]; int m32sn[4]; };
  typedef DecQ6K::Raw Raw;
  __device__ static void fill_lds(uint32_t*, uint32_t, uint32_t) {}
  struct TblRegs {};
  __device__ static TblRegs issue_tables(uint32_t, uint32_t) { return {}; }
  __device__ static void finish_tables(uint32_t*, const TblRegs&, uint32_t, uint32_t) {}

  __device__ static int byte_sums(uint32_t lo0, uint32_t lo1, uint32_t hi0, uint32_t hi1) {
    const int ones = 0x01010101;
    int sl = __builtin_amdgcn_sdot4((int)lo0, ones, 0, false);
    sl = __builtin_amdgcn_sdot4((int)lo1, ones, sl, false);
    int sh = __builtin_amdgcn_sdot4((int)hi0, ones, 0, false);
    sh = __builtin_amdgcn_sdot4((int)hi1, ones, sh, false);
    return (sh << 8) + sl;
  }
  // from the workgroup's staged, quantized row (units of kXqWords words per 32 consecutive columns)
  __device__ static X load_x(XQLds x, uint32_t u) {
    X r;
    const uint32_t j = u & 7u;
    const uint32_t xu0 = 8u * (u >> 3) + 4u * (j >> 2), w0 = 2u * (j & 3u);
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t* p = x.p + (xu0 + k) * kXqWords;
      const uint2 l = *(const uint2*)(p + w0), h = *(const uint2*)(p + 8u + w0);
      r.lo[2 * k] = l.x; r.lo[2 * k + 1] = l.y; r.hi[2 * k] = h.x; r.hi[2 * k + 1] = h.y;
      r.xs[k] = 8.f * __builtin_bit_cast(float, p[16]);  // the staged word holds an eighth of the scale
      r.m32sn[k] = -32 * byte_sums(l.x, l.y, h.x, h.y);
    }
    return r;
  }
  // the same quantization by one lane on its own (rows too long to stage; the decode matvec, from plain memory or the
  // padded LDS rows of XLds): one scale per run of eight columns
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    X r;
    const uint32_t j = u & 7u;
    const uint32_t base = 256u * (u >> 3) + 128u * (j >> 2) + 8u * (j & 3u);
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const float4* p = (const float4*)xat(x, base + 32u * k);
      const float4 a = p[0], b = p[1];
      const float m = fmaxf(fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))),
                            fmaxf(fmaxf(fabsf(b.x), fabsf(b.y)), fmaxf(fabsf(b.z), fabsf(b.w))));
      const int e = xq_exponent(m);
      const float mult = __builtin_ldexpf(kXqShrink, -e);
      xq_quant4(a, mult, r.lo[2 * k], r.hi[2 * k]);
      xq_quant4(b, mult, r.lo[2 * k + 1], r.hi[2 * k + 1]);
      r.xs[k] = __builtin_ldexpf(kXqUnit, e);
      r.m32sn[k] = -32 * byte_sums(r.lo[2 * k], r.lo[2 * k + 1], r.hi[2 * k], r.hi[2 * k + 1]);
    }
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) { return DecQ6K::load(row, u); }

  __device__ static float dot(const Raw& r, const X& x, const uint32_t*, uint32_t u) {
    // the lane's four scale bytes 2 k + is, is = (8 (j & 3)) / 16 the half of the run pair's 16-column scale group,
    // gathered into one word: each is then converted by a byte-select, without a shift of its own
    const uint32_t sc4 = __builtin_amdgcn_perm(r.sc[1], r.sc[0], (u & 2u) ? 0x07050301u : 0x06040200u);
    float total = 0.f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
      int lo = 0, hi = 0;
#pragma unroll
      for (int w = 0; w < 2; w++) {
        const uint32_t src = (k & 1) ? r.qb[w] : r.qa[w];
        const uint32_t n = (src >> (4 * (k >> 1))) & 0x0F0F0F0Fu;
        const uint32_t hb = 2 * k < 4 ? r.qh[w] << (4 - 2 * k) : r.qh[w] >> (2 * k - 4);
        const uint32_t q = (hb & 0x30303030u) | n;  // 4 bytes in 0..63
        if (w == 0) { lo = sdot4z(q, x.lo[2 * k]); hi = sdot4z(q, x.hi[2 * k]); }
        else {
          lo = __builtin_amdgcn_sdot4((int)q, (int)x.lo[2 * k + w], lo, false);
          hi = __builtin_amdgcn_sdot4((int)q, (int)x.hi[2 * k + w], hi, false);
        }
      }
      const float sc = (float)(int)(int8_t)(sc4 >> (8 * k));
      const float s = (float)((hi << 8) + lo + x.m32sn[k]);  // sum (q - 32) n: |.| < 2^24, exact
      total = __builtin_fmaf(sc, s * x.xs[k], total);
    }
    return half_bits_to_float(r.d) * total;
  }
};

}  // namespace msq
