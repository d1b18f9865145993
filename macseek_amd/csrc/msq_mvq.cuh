// Integer decoders of the decode matvec (one token): the block formats' dot products over activations quantized to 16-bit
// block-fixed-point integers (msq_iq1s.cuh: x ~ xs * n, |n| <= 32639, xs a power of two times a constant per run of
// columns), so that a single token's matvec rounds x at 2^-16 of its run's largest value instead of to fp16's 11 bits:
// the reference's one-token kernels take x as F32 and its test holds 2e-5 of sum |w x| (tests/test_quant_matvec.mm:42),
// which fp16 activations miss on rows shorter than about 9000 columns. Weights stay exact: integer payloads, scales
// applied in fp32. The several-token kernels keep the fp16 decoders of msq_device.cuh, like the reference's.
//
// Every decoder here quantizes its activation slice in the lane (load_x from plain memory or from a workgroup's padded
// LDS row), one scale per run of consecutive columns that shares a weight scale, and implements the interface of the
// fp16 decoder whose block layout, lane / unit mapping and loads it reuses.
#pragma once
#include "msq_iq2xxsq.cuh"
#include "msq_q6kq.cuh"

namespace msq {

typedef short s16x2_t __attribute__((ext_vector_type(2)));

// N4 x 4 consecutive activations (one scale): low / high byte words, the scale xs and the integer sum of the run
template <int N4, class S>
__device__ __forceinline__ void xq_run(S x, uint32_t col, uint32_t* lo, uint32_t* hi, float& xs, int& sn) {
  const float4* p = (const float4*)xat(x, col);
  float4 v[N4];
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < N4; i++) {
    v[i] = p[i];
    m = fmaxf(m, fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w))));
  }
  const int e = xq_exponent(m);
  const float mult = __builtin_ldexpf(kXqShrink, -e);
  int sl = 0, sh = 0;
#pragma unroll
  for (int i = 0; i < N4; i++) {
    xq_quant4(v[i], mult, lo[i], hi[i]);
    sl = __builtin_amdgcn_sdot4((int)lo[i], 0x01010101, sl, false);
    sh = __builtin_amdgcn_sdot4((int)hi[i], 0x01010101, sh, false);
  }
  xs = __builtin_ldexpf(kXqUnit, e);
  sn = (sh << 8) + sl;
}

// ------------------------------------------------------------------------------------------------ IQ1_S
// Grid entries as eight trit bytes (-1, 0, +1), two copies (copy c = lane & 1 of entry i at LDS byte (i << 4) | (c << 3)),
// then DecIQ1S's sixteen {2 s + 1, delta (2 s + 1)} pairs; sum w x = d ((2 s + 1) xs sum g n + delta (2 s + 1) xs sum n).
struct TblIQ1S8g { uint32_t w[MSQ_IQ1S_GRID_N * 2]; };
constexpr TblIQ1S8g make_iq1s8g() {
  TblIQ1S8g t{};
  for (int i = 0; i < MSQ_IQ1S_GRID_N; i++) {
    unsigned c = msq_iq1s_code[i];
    for (int j = 0; j < 8; j++, c /= 3) t.w[2 * i + j / 4] |= (uint32_t)(uint8_t)(int8_t)((int)(c % 3) - 1) << (8 * (j % 4));
  }
  return t;
}
__device__ __attribute__((aligned(16))) const TblIQ1S8g g_tbl_iq1s8g = make_iq1s8g();

struct DecIQ1SM {
  static constexpr int UNIT = 32, GRID_WORDS = MSQ_IQ1S_GRID_N * 4, LDS_WORDS = GRID_WORDS + 32;
  static constexpr uint32_t BLOCK = 50, UPB = 8;
  static constexpr bool STAGE_X = true;
  static constexpr int STAGES = 1;
  struct X { uint32_t lo[8], hi[8]; float xs, sx; };  // sx = xs * sum n: the sum of the unit's (rounded) activations
  typedef DecIQ1S::Raw Raw;
  typedef DecIQ1S::Off Off;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) {
    for (int i = tid; i < MSQ_IQ1S_GRID_N / 2; i += nt) {  // two entries per 16-byte item, each into both copies
      const u32x4 v = ((const u32x4*)g_tbl_iq1s8g.w)[i];
      *(u32x4*)(lds + 8 * i) = u32x4{v.x, v.y, v.x, v.y};
      *(u32x4*)(lds + 8 * i + 4) = u32x4{v.z, v.w, v.z, v.w};
    }
    for (int i = tid; i < 32; i += nt) lds[GRID_WORDS + i] = g_tbl_iq1s.w[MSQ_IQ1S_GRID_N * 4 + i];
  }
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    X r;
    int sn;
    xq_run<8>(x, 32u * u, r.lo, r.hi, r.xs, sn);
    r.sx = r.xs * (float)sn;
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) { return DecIQ1S::load(row, u); }
  __device__ static Off offsets(uint32_t u) { return DecIQ1S::offsets(u); }
  __device__ static Raw fetch(rsrc_t rs, const Off& o, uint32_t soff) { return DecIQ1S::fetch(rs, o, soff); }
  struct Look { uint2 g[4]; float2 f; };
  __device__ static Look lookup(const Raw& r, int, const uint32_t* lds) {
    const uint8_t* t = (const uint8_t*)lds;
    const uint32_t c = (threadIdx.x & 1u) << 3;
    Look k;
    k.f = *(const float2*)(t + GRID_WORDS * 4 + ((r.qh >> 9) & 0x78u));
#pragma unroll
    for (int l = 0; l < 4; l++) {
      const uint32_t off = (((r.qs >> (8 * l)) & 0xFFu) << 4) | (((r.qh >> (3 * l)) & 7u) << 12) | c;
      k.g[l] = *(const uint2*)(t + off);
    }
    return k;
  }
  __device__ static float partial(const Raw& r, const Look& k, const X& x, int, float) {
    int lo = 0, hi = 0, lo1 = 0, hi1 = 0;  // two interleaved pairs of chains
#pragma unroll
    for (int l = 0; l < 4; l += 2) {
      lo = __builtin_amdgcn_sdot4((int)k.g[l].x, (int)x.lo[2 * l], lo, false);
      hi = __builtin_amdgcn_sdot4((int)k.g[l].x, (int)x.hi[2 * l], hi, false);
      lo1 = __builtin_amdgcn_sdot4((int)k.g[l + 1].x, (int)x.lo[2 * l + 2], lo1, false);
      hi1 = __builtin_amdgcn_sdot4((int)k.g[l + 1].x, (int)x.hi[2 * l + 2], hi1, false);
      lo = __builtin_amdgcn_sdot4((int)k.g[l].y, (int)x.lo[2 * l + 1], lo, false);
      hi = __builtin_amdgcn_sdot4((int)k.g[l].y, (int)x.hi[2 * l + 1], hi, false);
      lo1 = __builtin_amdgcn_sdot4((int)k.g[l + 1].y, (int)x.lo[2 * l + 3], lo1, false);
      hi1 = __builtin_amdgcn_sdot4((int)k.g[l + 1].y, (int)x.hi[2 * l + 3], hi1, false);
    }
    const float acc = (float)(((hi + hi1) << 8) + lo + lo1) * x.xs;  // sum g x over the unit (the integer sum is exact)
    return half_bits_to_float(r.d) * __builtin_fmaf(k.f.x, acc, k.f.y * x.sx);
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t* lds) { return partial(r, lookup(r, 0, lds), x, 0, 0.f); }
};

// ------------------------------------------------------------------------------------------------ IQ2_XXS
// DecIQ2XXSQ with compact tables (12 KB instead of a 64 KB region: several matvec workgroups share a CU): grid entry e,
// copy c = lane & 3, at LDS byte (e << 5) | (c << 3); sign entry i, copy c = lane & 1, at 8192 + ((i << 5) | (c << 4)).
struct DecIQ2XXSM : DecIQ2XXSQ {
  static constexpr int LDS_WORDS = 3072;
  static constexpr int SIGN_AT = 8192;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) {
    uint8_t* t = (uint8_t*)lds;
    for (int i = tid; i < 256; i += nt) {
      const u32x4 v = ((const u32x4*)g_tbl_iq2xxs8.w)[i];
      if (i < 128) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          *(uint2*)(t + ((2 * i) << 5) + (c << 3)) = uint2{v.x, v.y};
          *(uint2*)(t + ((2 * i + 1) << 5) + (c << 3)) = uint2{v.z, v.w};
        }
      } else {
#pragma unroll
        for (int c = 0; c < 2; c++) *(u32x4*)(t + SIGN_AT + ((i - 128) << 5) + (c << 4)) = v;
      }
    }
  }
  __device__ static Look lookup(const Raw& r, int stage, const uint32_t* lds) {
    const uint8_t* t = (const uint8_t*)lds;
    const uint32_t cg = (threadIdx.x & 3u) << 3, cs = SIGN_AT | ((threadIdx.x & 1u) << 4);
    Look k;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int l = 2 * stage + i;
      const uint32_t ag = (((r.a0 >> (8 * l)) & 0xFFu) << 5) | cg;
      const uint32_t as = (((r.a1 >> (7 * l)) & 127u) << 5) | cs;
      k.g[i] = *(const uint2*)(t + ag);
      k.s[i] = *(const u32x4*)(t + as);
    }
    return k;
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t* lds) {
    const Look k0 = lookup(r, 0, lds), k1 = lookup(r, 1, lds);
    return partial(r, k1, x, 1, partial(r, k0, x, 0, 0.f));
  }
};

// ------------------------------------------------------------------------------------------------ Q5_K
// DecQ5K's mapping: unit j of a block owns two runs of 16 columns, 64 (j >> 1) + 16 (j & 1) + 32 run, each with its own
// 6-bit scale and min: sum w x = d sc xs_run sum q n - dmin m xs_run sum n, q = nibble | high bit << 4 in 0..31.
struct DecQ5KQ {
  static constexpr int UNIT = 32, LDS_WORDS = 0;
  static constexpr uint32_t BLOCK = 176, UPB = 8;
  static constexpr bool STAGE_X = false;
  struct X { uint32_t lo[8], hi[8]; float xs[2], sx[2]; };
  typedef DecQ5K::Raw Raw;
  __device__ static void fill_lds(uint32_t*, int, int) {}
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    X r;
    const uint32_t j = u & 7u;
    const uint32_t base = 256u * (u >> 3) + 64u * (j >> 1) + 16u * (j & 1u);
#pragma unroll
    for (int run = 0; run < 2; run++) {
      int sn;
      xq_run<4>(x, base + 32u * run, r.lo + 4 * run, r.hi + 4 * run, r.xs[run], sn);
      r.sx[run] = r.xs[run] * (float)sn;
    }
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) { return DecQ5K::load(row, u); }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t*, uint32_t u) {
    const uint32_t g = (u & 7u) >> 1;
    const float d = half_bits_to_float(r.dd & 0xFFFFu), dmin = half_bits_to_float(r.dd >> 16);
    float total = 0.f;
#pragma unroll
    for (int run = 0; run < 2; run++) {
      int lo = 0, hi = 0;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        const uint32_t n = (r.ql[w] >> (4 * run)) & 0x0F0F0F0Fu;
        const uint32_t hb = ((r.qh[w] >> (2 * g + run)) & 0x01010101u) << 4;
        const uint32_t q = n | hb;  // 4 bytes in 0..31
        if (w == 0) { lo = sdot4z(q, x.lo[4 * run]); hi = sdot4z(q, x.hi[4 * run]); }
        else {
          lo = __builtin_amdgcn_sdot4((int)q, (int)x.lo[4 * run + w], lo, false);
          hi = __builtin_amdgcn_sdot4((int)q, (int)x.hi[4 * run + w], hi, false);
        }
      }
      const uint32_t a = (r.pa >> (8 * run)) & 0xFFu, bq = (r.pb >> (8 * run)) & 0xFFu, c = (r.pc >> (8 * run)) & 0xFFu;
      uint32_t sc, mn;
      if (g < 2) { sc = a & 63u; mn = bq & 63u; }
      else { sc = (bq & 0xFu) | ((c >> 6) << 4); mn = (bq >> 4) | ((a >> 6) << 4); }
      const float acc = (float)((hi << 8) + lo) * x.xs[run];  // |integer sum| < 2^24: exact
      total += (d * (float)sc) * acc - (dmin * (float)mn) * x.sx[run];
    }
    return total;
  }
};

// ------------------------------------------------------------------------------------------------ IQ4_NL
// A byte of qs holds the codebook indices of columns j (low nibble) and j + 16 (high nibble): the table turns it into
// the two int16 values, and one v_dot2_i32_i16 multiplies them with the activations' 16-bit integers of the same two
// columns (pairs (n_j, n_{j + 16}), as DecIQ4NL keeps its fp16 pairs).
struct TblIQ4NL16 { uint32_t w[256]; };
constexpr TblIQ4NL16 make_iq4nl16() {
  TblIQ4NL16 t{};
  for (int b = 0; b < 256; b++)
    t.w[b] = (uint32_t)(uint16_t)(int16_t)kIQ4NLValues[b & 15] | ((uint32_t)(uint16_t)(int16_t)kIQ4NLValues[b >> 4] << 16);
  return t;
}
__device__ __attribute__((aligned(16))) const TblIQ4NL16 g_tbl_iq4nl16 = make_iq4nl16();

struct DecIQ4NLQ {
  static constexpr int UNIT = 32, LDS_WORDS = 256;
  static constexpr uint32_t BLOCK = 18, UPB = 1;
  static constexpr bool STAGE_X = true;
  struct X { uint32_t v[16]; float xs; };  // pair j = (n[j], n[j + 16]) as int16
  typedef DecIQ4NL::Raw Raw;
  __device__ static void fill_lds(uint32_t* lds, int tid, int nt) { copy_words16(lds, g_tbl_iq4nl16.w, 256, tid, nt); }
  template <class S>
  __device__ static X load_x(S x, uint32_t u) {
    X r;
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
    auto pair = [&](float a, float b) { return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pknorm_i16(a * mult, b * mult)); };
#pragma unroll
    for (int i = 0; i < 4; i++) {
      r.v[4 * i] = pair(v[i].x, v[i + 4].x); r.v[4 * i + 1] = pair(v[i].y, v[i + 4].y);
      r.v[4 * i + 2] = pair(v[i].z, v[i + 4].z); r.v[4 * i + 3] = pair(v[i].w, v[i + 4].w);
    }
    r.xs = __builtin_ldexpf(kXqUnit, e);
    return r;
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) { return DecIQ4NL::load(row, u); }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t* lds) {
    int acc = 0, acc1 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int k = 0; k < 4; k += 2) {
        acc = __builtin_amdgcn_sdot2(__builtin_bit_cast(s16x2_t, lds[(r.q[i] >> (8 * k)) & 0xFFu]), __builtin_bit_cast(s16x2_t, x.v[4 * i + k]), acc, false);
        acc1 = __builtin_amdgcn_sdot2(__builtin_bit_cast(s16x2_t, lds[(r.q[i] >> (8 * k + 8)) & 0xFFu]), __builtin_bit_cast(s16x2_t, x.v[4 * i + k + 1]), acc1, false);
      }
    }
    return half_bits_to_float(r.d) * ((float)(acc + acc1) * x.xs);  // |integer sum| < 2^28: the conversion rounds at 2^-24
  }
};

}  // namespace msq
