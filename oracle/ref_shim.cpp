// C entry points over the reference's own CPU dequant (tests/ref/dequant.cpp), compiled from /root/reference where
// it lies. Used only to validate oracle.c and to write the golden fixtures; never shipped, never on the GPU box.
#include <cstring>
#include <vector>
#include "ref/dequant.hpp"

extern "C" {
void refshim_dequant_row(int t, const void* src, float* dst, long long n) {
  ref::dequant_row((ref::QType)t, src, dst, n);
}
void refshim_matvec(int t, const void* W, int rows, int cols, const float* x, float* y) {
  ref::matvec_ref((ref::QType)t, W, rows, cols, x, y);
}
unsigned short refshim_f32_to_fp16(float f) { return ref::f32_to_fp16(f); }
float refshim_fp16_to_f32(unsigned short h) { return ref::fp16_to_f32(h); }
}
