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

// The reference's router / route-list CPU twins (tests/ref/arch_ref.cpp:97-130), built into _ref/libref_arch.so.
#ifdef REFSHIM_ARCH
#include "ref/arch_ref.hpp"
extern "C" {
void refshim_router(const float* logits, const float* bias, int* ids, float* w, float route_scale) {
  ref_arch::router(logits, bias, ids, w, route_scale);
}
void refshim_rmsnorm(const float* x, const float* w, float* y, int dim, double eps) { ref_arch::rmsnorm(x, w, y, dim, eps); }
void refshim_route_lists(const int* ids, const float* w, int n, unsigned* counts, unsigned* offsets, unsigned* entry,
                         unsigned* tok, float* lw, unsigned* slot_of) {
  std::vector<uint32_t> c, o, e, t, s;
  std::vector<float> l;
  ref_arch::route_lists(ids, w, n, c, o, e, t, l, s);
  memcpy(counts, c.data(), c.size() * 4); memcpy(offsets, o.data(), o.size() * 4);
  memcpy(entry, e.data(), e.size() * 4); memcpy(tok, t.data(), t.size() * 4);
  memcpy(lw, l.data(), l.size() * 4); memcpy(slot_of, s.data(), s.size() * 4);
}
}
#endif
