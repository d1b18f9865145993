// IQ2_XXS decoder for the gate/up kernel of the one-token MoE layer: integer dot products over the 16-bit
// block-fixed-point activations of msq_iq1s.cuh (the fp16 decoder DecIQ2XXS rounds x to 11 significant bits; on a
// shared expert, whose weight is 1, that rounding alone is the layer's whole error against an F32-activation
// reference: 1.2e-4 of sum |w h| on the 7168 / 2048 layer, 2e-5 with the activations of this file).
//
// Block layout {fp16 d; u16 qs[32]} and the arithmetic w = d (0.5 + s) 0.25 grid sign follow the reference's CPU
// dequantizer (tests/ref/dequant.cpp:92-106): per 32 weights eight bytes, a0 = four grid indices, a1 = four 7-bit sign
// indices and the 4-bit scale s. What is this library's own:
//   * the grid magnitudes 8 / 25 / 43 stay bytes; a sign index delivers a byte mask M (0xFF where the weight is
//     negative) and C = M & 0x01010101, and (m ^ M) + C negates the masked bytes in one instruction per four weights
//     (m >= 8, so no byte carries into its neighbour); a unit's dot product is then 16 v_dot4_i32_i8 against the low and
//     the high byte plane of the activations;
//   * tables at a 256-byte pitch, so that a lookup address is a byte permutation: grid entry b, copy c = lane & 15, at
//     LDS byte (b << 8) | (c << 3); sign entry i, copy c = lane & 7, at (i << 8) | 128 | (c << 4). Lanes of different
//     copies never meet in a bank; the sixteen / eight lanes that share a copy spread over all banks.
#pragma once
#include "msq_iq1s.cuh"

namespace msq {

// image: 256 grid entries of 8 magnitude bytes, then 128 sign entries {M lo, M hi, C lo, C hi}
struct TblIQ2XXS8 { uint32_t w[MSQ_IQ2XXS_GRID_N * 2 + 128 * 4]; };
constexpr TblIQ2XXS8 make_iq2xxs8() {
  TblIQ2XXS8 t{};
  constexpr uint32_t mag[3] = {8, 25, 43};
  for (int i = 0; i < MSQ_IQ2XXS_GRID_N; i++) {
    unsigned c = msq_iq2xxs_code[i];
    for (int j = 0; j < 8; j++, c /= 3) t.w[2 * i + j / 4] |= mag[c % 3] << (8 * (j % 4));
  }
  for (int i = 0; i < 128; i++) {  // ksigns_iq2xs[i] = i | parity(i) << 7; bit j set: element j is negative
    int par = 0;
    for (int b = 0; b < 7; b++) par ^= (i >> b) & 1;
    const unsigned s = (unsigned)i | ((unsigned)par << 7);
    uint32_t* e = t.w + MSQ_IQ2XXS_GRID_N * 2 + 4 * i;
    for (int j = 0; j < 8; j++)
      if ((s >> j) & 1) { e[j / 4] |= 0xFFu << (8 * (j % 4)); e[2 + j / 4] |= 1u << (8 * (j % 4)); }
  }
  return t;
}
__device__ __attribute__((aligned(16))) const TblIQ2XXS8 g_tbl_iq2xxs8 = make_iq2xxs8();

struct DecIQ2XXSQ {
  static constexpr int UNIT = 32;
  static constexpr uint32_t BLOCK = 66, UPB = 8;
  static constexpr int LDS_WORDS = 16384;  // 256 rows of 256 bytes
  static constexpr bool STAGE_X = true, QUANT_X = true;
  static constexpr int STAGES = 2;         // two grid entries (16 weights) per stage
  typedef DecIQ1SQ::X X;                   // the unit's low / high byte planes and an eighth of its scale
  struct Raw { uint32_t a0, a1; _Float16 d; };

  // ---- tables: 256 16-byte items of the image (128 x two grid entries, 128 x one sign entry); work piece i = item
  // (i & 255), quarter (i >> 8) of its copies. issue_tables requests the thread's first item, finish_tables stores.
  static constexpr uint32_t ITEMS = 256, PIECES = 4 * ITEMS;
  struct TblRegs { u32x4 v; };
  __device__ static TblRegs issue_tables(uint32_t tid, uint32_t) { return {((const u32x4*)g_tbl_iq2xxs8.w)[tid & 255u]}; }
  __device__ static void finish_tables(uint32_t* lds, const TblRegs& r, uint32_t tid, uint32_t nt) {
    uint8_t* t = (uint8_t*)lds;
    auto put = [&](uint32_t i, const u32x4& v) {
      const uint32_t item = i & 255u, quarter = i >> 8;
      if (item < 128u) {  // grid entries 2 item, 2 item + 1: copies 4 quarter .. 4 quarter + 3
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const uint32_t at = (4u * quarter + c) << 3;
          *(uint2*)(t + ((2u * item) << 8) + at) = uint2{v.x, v.y};
          *(uint2*)(t + ((2u * item + 1u) << 8) + at) = uint2{v.z, v.w};
        }
      } else {            // sign entry item - 128: copies 2 quarter, 2 quarter + 1
#pragma unroll
        for (int c = 0; c < 2; c++) *(u32x4*)(t + ((item - 128u) << 8) + 128u + ((2u * quarter + c) << 4)) = v;
      }
    };
    if (tid < PIECES) put(tid, r.v);
    uint32_t t2 = tid;
    asm volatile("" : "+v"(t2));  // (addresses of a loop that rarely runs stay out of the prologue's registers)
    for (uint32_t i = t2 + nt; i < PIECES; i += nt) put(i, ((const u32x4*)g_tbl_iq2xxs8.w)[i & 255u]);
  }
  __device__ static void fill_lds(uint32_t* lds, uint32_t tid, uint32_t nt) { finish_tables(lds, issue_tables(tid, nt), tid, nt); }

  // ---- activations: as DecIQ1SQ
  __device__ static X load_x(XQLds x, uint32_t u) { return DecIQ1SQ::load_x(x, u); }
  template <class S>
  __device__ static X load_x(S x, uint32_t u) { return DecIQ1SQ::load_x(x, u); }

  // ---- block bytes
  struct Off { uint32_t a, d; };
  __device__ static Off offsets(uint32_t u) {
    const uint32_t b = (u >> 3) * 66u;
    return {b + 2 + 8 * (u & 7u), b};
  }
  __device__ static Raw fetch(rsrc_t rs, const Off& o, uint32_t soff) {
    const u64_a2 a = buf_ld64(rs, o.a, soff);
    return {a.x, a.y, __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(rs, (int)o.d, (int)soff, 0))};
  }

  // ---- decode: lookup() issues the table reads of a stage, partial() consumes them
  struct Look { uint2 g[2]; u32x4 s[2]; };
  __device__ static Look lookup(const Raw& r, int stage, const uint32_t* lds) {
    const uint8_t* t = (const uint8_t*)lds;
    const uint32_t lane = threadIdx.x;  // the copies are lane & 15 / lane & 7
    const uint32_t cg = (lane & 15u) << 3, cs = 128u | ((lane & 7u) << 4);
    Look k;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int l = 2 * stage + i;
      // grid: byte l of a0 becomes address byte 1
      const uint32_t ag = __builtin_amdgcn_perm(r.a0, cg, 0x0c0c0400u + ((uint32_t)l << 8));
      // sign index (a1 >> 7 l) & 127 moved to bits 8..14
      const uint32_t sh = 7 * l < 8 ? r.a1 << (8 - 7 * l) : r.a1 >> (7 * l - 8);
      const uint32_t as = (sh & 0x7F00u) | cs;
      k.g[i] = *(const uint2*)(t + ag);
      k.s[i] = *(const u32x4*)(t + as);
    }
    return k;
  }
  // sum over the stage's 16 weights of (+- magnitude) * n, n = 256 nh + nl the activation's integer
  __device__ static float stage_sum(const Look& k, const X& x, int stage) {
    int lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int l = 2 * stage + i;
      // (m ^ M) + C: the bytes under the mask negated
      uint32_t w0, w1;
      asm("v_xad_u32 %0, %1, %2, %3" : "=v"(w0) : "v"(k.g[i].x), "v"(k.s[i].x), "v"(k.s[i].z));
      asm("v_xad_u32 %0, %1, %2, %3" : "=v"(w1) : "v"(k.g[i].y), "v"(k.s[i].y), "v"(k.s[i].w));
      lo = __builtin_amdgcn_sdot4((int)w0, (int)x.lo[2 * l], lo, false);
      hi = __builtin_amdgcn_sdot4((int)w0, (int)x.hi[2 * l], hi, false);
      lo = __builtin_amdgcn_sdot4((int)w1, (int)x.lo[2 * l + 1], lo, false);
      hi = __builtin_amdgcn_sdot4((int)w1, (int)x.hi[2 * l + 1], hi, false);
    }
    return (float)((hi << 8) + lo);  // |sum| < 2^25: the conversion rounds at 2^-24 of it
  }
  template <class P>
  __device__ static Raw load(P row, uint32_t u) {
    const P b = row + (u >> 3) * 66u;
    const u64_a2 a = ld64(b + 2 + 8 * (u & 7u));
    return {a.x, a.y, __builtin_bit_cast(_Float16, (uint16_t)ld16(b))};
  }
  __device__ static float dot(const Raw& r, const X& x, const uint32_t* lds) {
    const Look k0 = lookup(r, 0, lds), k1 = lookup(r, 1, lds);
    return partial(r, k1, x, 1, partial(r, k0, x, 0, 0.f));
  }
  __device__ static float partial(const Raw& r, const Look& k, const X& x, int stage, float acc) {
    acc += stage_sum(k, x, stage);
    if (stage == STAGES - 1) {
      // d (2 s + 1) / 8 * xs * sum = d * (2 s + 1) * xs8 * sum
      const float f = (float)(((r.a1 >> 27) & 0x1Eu) | 1u);
      const float w = (acc * x.xs8) * f;
      asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(acc) : "v"(r.d), "v"(w));  // the fp16 d converted inside the multiply
    }
    return acc;
  }
};

}  // namespace msq
