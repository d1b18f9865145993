// Quant type ids and block geometry shared by host and device code. Ids equal the ggml type ids, so a GGUF type field
// maps 1:1 (reference: src/kernels/quant_types.hpp:8-43).
#pragma once
#include <stddef.h>
#include <stdint.h>

enum MsqType : int {
  MSQ_F32 = 0, MSQ_F16 = 1, MSQ_Q8_0 = 8, MSQ_Q5_K = 13, MSQ_Q6_K = 14, MSQ_IQ2_XXS = 16, MSQ_IQ1_S = 19,
  MSQ_IQ4_NL = 20, MSQ_BF16 = 30
};

static inline int msq_type_block_elems(int t) {
  switch (t) {
    case MSQ_F32: case MSQ_F16: case MSQ_BF16: return 1;
    case MSQ_Q8_0: case MSQ_IQ4_NL: return 32;
    case MSQ_Q5_K: case MSQ_Q6_K: case MSQ_IQ2_XXS: case MSQ_IQ1_S: return 256;
    default: return 0;
  }
}
static inline size_t msq_type_block_bytes(int t) {
  switch (t) {
    case MSQ_F32: return 4;
    case MSQ_F16: case MSQ_BF16: return 2;
    case MSQ_Q8_0: return 34;
    case MSQ_Q5_K: return 176;
    case MSQ_Q6_K: return 210;
    case MSQ_IQ2_XXS: return 66;
    case MSQ_IQ1_S: return 50;
    case MSQ_IQ4_NL: return 18;
    default: return 0;
  }
}
static inline size_t msq_type_row_bytes(int t, int64_t cols) {
  const int be = msq_type_block_elems(t);
  return be ? (size_t)(cols / be) * msq_type_block_bytes(t) : 0;
}
static inline const char* msq_type_name_of(int t) {
  switch (t) {
    case MSQ_F32: return "F32"; case MSQ_F16: return "F16"; case MSQ_BF16: return "BF16";
    case MSQ_Q8_0: return "Q8_0"; case MSQ_Q5_K: return "Q5_K"; case MSQ_Q6_K: return "Q6_K";
    case MSQ_IQ2_XXS: return "IQ2_XXS"; case MSQ_IQ1_S: return "IQ1_S"; case MSQ_IQ4_NL: return "IQ4_NL";
    default: return "?";
  }
}
