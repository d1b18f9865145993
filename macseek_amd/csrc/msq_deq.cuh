// Whole-buffer dequantization to fp32, bit-exact with the reference CPU dequantizer: every expression keeps the
// operand order of tests/ref/dequant.cpp:34-120 and floating-point contraction is off, so no multiply-subtract fuses.
// One thread produces 8 consecutive elements.
#pragma once
#include "msq_device.cuh"

namespace msq {

__device__ __forceinline__ float tbl_half(const uint32_t* w, int j) {  // element j of an 8-half table entry
  const uint32_t v = w[j >> 1];
  return half_bits_to_float((j & 1) ? (v >> 16) : (v & 0xFFFFu));
}

// OUT = float: the bit-exact fp32 result. OUT = uint16_t: the same values rounded to fp16 (nearest even), the weight
// operand of the prefill matmul (reference: q_deq_f16, src/kernels/quant_mm.metal:143-154).
template <int QT, class OUT = float>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ src, OUT* __restrict__ dst, int64_t nchunks) {
#pragma clang fp contract(off)
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= nchunks) return;
  float y[8];
  if constexpr (QT == MSQ_F32) {
    for (int j = 0; j < 8; j++) y[j] = __builtin_bit_cast(float, ld32(src + 4 * (8 * c + j)));
  } else if constexpr (QT == MSQ_F16) {
    for (int j = 0; j < 8; j++) y[j] = half_bits_to_float(ld16(src + 2 * (8 * c + j)));
  } else if constexpr (QT == MSQ_BF16) {
    for (int j = 0; j < 8; j++) y[j] = bf16_bits_to_float(ld16(src + 2 * (8 * c + j)));
  } else if constexpr (QT == MSQ_Q8_0) {  // dequant.cpp:40-45
    const uint8_t* b = src + (c >> 2) * 34;
    const float d = half_bits_to_float(ld16(b));
    const uint8_t* q = b + 2 + 8 * (c & 3);
    for (int j = 0; j < 8; j++) y[j] = (float)(int8_t)q[j] * d;
  } else if constexpr (QT == MSQ_IQ4_NL) {  // dequant.cpp:107-112
    const uint8_t* b = src + (c >> 2) * 18;
    const float d = half_bits_to_float(ld16(b));
    const int part = (int)(c & 3);
    const uint8_t* q = b + 2 + 8 * (part & 1);
    for (int j = 0; j < 8; j++) {
      const int nib = part < 2 ? (q[j] & 0xF) : (q[j] >> 4);
      y[j] = d * half_bits_to_float(g_tbl_iq4nl.w[nib] & 0xFFFFu);  // low half of entry b = kv[b & 15]
    }
  } else if constexpr (QT == MSQ_IQ1_S) {  // dequant.cpp:77-91
    const uint8_t* b = src + (c >> 5) * 50;
    const int r = (int)(c & 31), ib = r >> 2, l = r & 3;
    const float d = half_bits_to_float(ld16(b));
    const uint32_t qh = ld16(b + 34 + 2 * ib);
    const float dl = d * (float)(2 * ((qh >> 12) & 7) + 1);
    const float delta = (qh & 0x8000) ? -0.125f : 0.125f;
    const uint32_t* g = g_tbl_iq1s.w + 4 * (b[2 + r] | (((qh >> (3 * l)) & 7) << 8));
    for (int j = 0; j < 8; j++) y[j] = dl * (tbl_half(g, j) + delta);
  } else if constexpr (QT == MSQ_IQ2_XXS) {  // dequant.cpp:92-106
    const uint8_t* b = src + (c >> 5) * 66;
    const int r = (int)(c & 31), ib = r >> 2, l = r & 3;
    const float d = half_bits_to_float(ld16(b));
    const uint8_t* a8 = b + 2 + 8 * ib;
    const uint32_t a1 = ld32(a8 + 4);
    const float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
    const uint32_t* g = g_tbl_iq2xxs.w + 4 * a8[l];
    const uint32_t si = (a1 >> (7 * l)) & 127u;
    const uint32_t sg = si | ((__builtin_popcount(si) & 1u) << 7);
    for (int j = 0; j < 8; j++) y[j] = db * tbl_half(g, j) * ((sg >> j) & 1u ? -1.f : 1.f);
  } else if constexpr (QT == MSQ_Q6_K) {  // dequant.cpp:60-76
    const uint8_t* b = src + (c >> 5) * 210;
    const int e0 = 8 * (int)(c & 31), h = e0 >> 7, k = (e0 & 127) >> 5, l0 = e0 & 31;
    const float d = half_bits_to_float(ld16(b + 208));
    const uint8_t* ql = b + 64 * h + ((k & 1) ? 32 : 0) + l0;
    const uint8_t* qh = b + 128 + 32 * h + l0;
    const float sc = (float)(int8_t)b[192 + 8 * h + (l0 >> 4) + 2 * k];
    for (int j = 0; j < 8; j++) {
      const int nib = (k >> 1) ? (ql[j] >> 4) : (ql[j] & 0xF);
      const int q = (nib | (((qh[j] >> (2 * k)) & 3) << 4)) - 32;
      y[j] = d * sc * (float)q;
    }
  } else if constexpr (QT == MSQ_Q5_K) {  // dequant.cpp:46-59, scale unpack :29-32
    const uint8_t* b = src + (c >> 5) * 176;
    const int e0 = 8 * (int)(c & 31), g = e0 >> 6, run = (e0 & 63) >> 5, l0 = e0 & 31, is = 2 * g + run;
    const float d = half_bits_to_float(ld16(b)), mn = half_bits_to_float(ld16(b + 2));
    const uint8_t* s = b + 4;
    uint32_t sc, m;
    if (is < 4) { sc = s[is] & 63u; m = s[is + 4] & 63u; }
    else { sc = (s[is + 4] & 0xFu) | ((uint32_t)(s[is - 4] >> 6) << 4); m = (uint32_t)(s[is + 4] >> 4) | ((uint32_t)(s[is] >> 6) << 4); }
    const float d1 = d * (float)sc, m1 = mn * (float)m;
    const uint8_t* ql = b + 48 + 32 * g + l0;
    const uint8_t* qh = b + 16 + l0;
    for (int j = 0; j < 8; j++) {
      const int nib = run ? (ql[j] >> 4) : (ql[j] & 0xF);
      const int q = nib + (((qh[j] >> (2 * g + run)) & 1) ? 16 : 0);
      y[j] = d1 * (float)q - m1;
    }
  }
  if constexpr (sizeof(OUT) == 4) {
    float4* o = (float4*)(dst + 8 * c);
    o[0] = make_float4(y[0], y[1], y[2], y[3]);
    o[1] = make_float4(y[4], y[5], y[6], y[7]);
  } else {
    *(uint4*)(dst + 8 * c) = uint4{pack_h2(y[0], y[1]), pack_h2(y[2], y[3]), pack_h2(y[4], y[5]), pack_h2(y[6], y[7])};
  }
}

}  // namespace msq
