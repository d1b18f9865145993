// C++20 shim: the reference's operator API (namespace ms::q, src/kernels/quant.hpp) over the libmsq C ABI.
//
// A caller written against the reference keeps its call sites: same function names, argument order and meaning. What
// changes is the runtime underneath -- ms::Enc wraps a hipStream_t instead of a Metal command encoder, ms::Buffer a
// device pointer instead of an MTLBuffer -- and two trailing members (dim, inter) on the MoE argument structs, which
// default to the reference's hard-coded expert shape (quant.hpp:49). Misuse behaves as in the reference: the message
// "macseek quant: ... unsupported (...)" goes to stderr and the process aborts (src/kernels/quant.mm:34-37).
#pragma once
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../msq.h"

namespace ms {

// reference: ms::Buffer (src/core/metal.hpp:11-18)
struct Buffer {
  void* buf = nullptr;  // device allocation
  size_t off = 0;
  size_t size = 0;
  Buffer sub(size_t o, size_t s) const { return Buffer{buf, off + o, s}; }
  MsqBuffer c() const { return MsqBuffer{buf, off, size}; }
};

// reference: ms::Enc (src/core/metal.hpp:37-71), reduced to what the quant operators use. The stream is in-order, so
// barrier() has nothing to do; wait() is left to the caller's runtime (hipStreamSynchronize on `stream`).
struct Enc {
  void* stream = nullptr;  // hipStream_t
  void barrier() {}
};

namespace q {

enum class QType : int {  // reference: src/kernels/quant_types.hpp:9-11
  F32 = 0, F16 = 1, Q8_0 = 8, Q5_K = 13, Q6_K = 14, IQ2_XXS = 16, IQ1_S = 19, IQ4_NL = 20, BF16 = 30, MXFP4 = 39,
};
inline int block_elems(QType t) { return msq_block_elems((int)t); }
inline size_t block_bytes(QType t) { return msq_block_bytes((int)t); }
inline size_t row_bytes(QType t, int64_t cols) { return msq_row_bytes((int)t, cols); }
inline const char* type_name(QType t) { return msq_type_name((int)t); }

namespace detail {
[[noreturn]] inline void die() {
  fprintf(stderr, "%s\n", msq_last_error());
  abort();
}
inline void check(int rc) { if (rc != MSQ_OK) die(); }
}  // namespace detail

struct MvCfg { int nr = 0, rsg = 0, ks = 0; };  // reference: quant.hpp:12

inline bool matvec_supported(QType t) { return msq_matvec_supported((int)t) != 0; }
inline MvCfg matvec_cfg(QType t, int rows, int cols) {
  MsqMvCfg c{};
  detail::check(msq_matvec_cfg((int)t, rows, cols, &c));
  return MvCfg{c.nr, c.rsg, c.ks};
}
inline void encode_matvec(Enc& e, QType t, const Buffer& W, int rows, int cols, const Buffer& x, const Buffer& y,
                          bool accumulate = false, int groups = 1, MvCfg cfg = {}) {
  const MsqBuffer w = W.c(), xb = x.c(), yb = y.c();
  const MsqMvCfg c{cfg.nr, cfg.rsg, cfg.ks};
  detail::check(msq_matvec(e.stream, (int)t, &w, rows, cols, &xb, &yb, accumulate, groups, &c));
}
// reference: quant.hpp:20-26
inline void encode_matvec_rmsnorm(Enc& e, QType t, const Buffer& W, int rows, int cols, const Buffer& x, const Buffer& norm_w,
                                  float eps, const Buffer& y, int tiles_per_tg = 0) {
  const MsqBuffer w = W.c(), xb = x.c(), nb = norm_w.c(), yb = y.c();
  detail::check(msq_matvec_rmsnorm(e.stream, (int)t, &w, rows, cols, &xb, &nb, eps, &yb, tiles_per_tg));
}
inline void encode_matvec_n(Enc& e, QType t, const Buffer& W, int rows, int cols, const Buffer& X, const Buffer& Y, int n,
                            bool accumulate = false, int groups = 1) {
  const MsqBuffer w = W.c(), xb = X.c(), yb = Y.c();
  detail::check(msq_matvec_n(e.stream, (int)t, &w, rows, cols, &xb, &yb, n, accumulate, groups));
}

// reference: quant.hpp:40-45
inline void encode_matmul(Enc& e, QType t, const Buffer& W, int rows, int cols, const Buffer& X, const Buffer& Y, int n,
                          bool accumulate = false) {
  const MsqBuffer w = W.c(), xb = X.c(), yb = Y.c();
  detail::check(msq_matmul(e.stream, (int)t, &w, rows, cols, &xb, &yb, n, accumulate));
}
inline void encode_f32_to_f16(Enc& e, const Buffer& X, const Buffer& X16, size_t count) {
  const MsqBuffer xb = X.c(), hb = X16.c();
  detail::check(msq_f32_to_f16(e.stream, &xb, &hb, count));
}
inline void encode_matmul_h(Enc& e, QType t, const Buffer& W, int rows, int cols, const Buffer& X16, const Buffer& Y, int n,
                            bool accumulate = false, int x_stride = 0) {
  const MsqBuffer w = W.c(), xb = X16.c(), yb = Y.c();
  detail::check(msq_matmul_h(e.stream, (int)t, &w, rows, cols, &xb, &yb, n, accumulate, x_stride));
}

// ---- MoE ----
constexpr int kExpertDim = MSQ_EXPERT_DIM, kExpertInter = MSQ_EXPERT_INTER, kMaxRouted = MSQ_MAX_ROUTED;

struct ExpertSlot {
  Buffer gate, up, down;
  MsqExpertSlot c() const { return MsqExpertSlot{gate.c(), up.c(), down.c()}; }
};

struct MoeDecodeArgs {  // reference: quant.hpp:55-71
  QType t_gate_up = QType::IQ1_S;
  QType t_down = QType::IQ1_S;
  int n_routed = 6;
  ExpertSlot slot[kMaxRouted];
  Buffer weights;
  bool has_shared = true;
  QType t_shared = QType::Q6_K;
  ExpertSlot shared;
  Buffer x, y, scratch;
  int gu_nr = 0, gu_rsg = 0, d_nr = 0, d_rsg = 0;
  int dim = kExpertDim, inter = kExpertInter;  // not in the reference: its expert shape is a compile-time constant
  MsqMoeDecodeArgs c() const {
    MsqMoeDecodeArgs a{};
    a.t_gate_up = (int)t_gate_up; a.t_down = (int)t_down; a.n_routed = n_routed;
    for (int i = 0; i < kMaxRouted; i++) a.slot[i] = slot[i].c();
    a.weights = weights.c(); a.has_shared = has_shared; a.t_shared = (int)t_shared; a.shared = shared.c();
    a.x = x.c(); a.y = y.c(); a.scratch = scratch.c();
    a.gu_nr = gu_nr; a.gu_rsg = gu_rsg; a.d_nr = d_nr; a.d_rsg = d_rsg; a.dim = dim; a.inter = inter;
    return a;
  }
};
inline size_t moe_decode_scratch_bytes(int inter = kExpertInter) { return msq_moe_decode_scratch_bytes(inter); }
inline void encode_moe_decode(Enc& e, const MoeDecodeArgs& a) {
  const MsqMoeDecodeArgs c = a.c();
  detail::check(msq_moe_decode(e.stream, &c));
}
inline void encode_moe_decode_table(Enc& e, const MoeDecodeArgs& a, const Buffer& table) {
  const MsqMoeDecodeArgs c = a.c();
  const MsqBuffer t = table.c();
  detail::check(msq_moe_decode_table(e.stream, &c, &t));
}
// no reference counterpart: the same layer with the h scratch in the library's static device array (nothing is
// allocated, a.scratch is ignored, inter <= msq_moe_decode_static_max_inter())
inline void encode_moe_decode_static(Enc& e, const MoeDecodeArgs& a) {
  const MsqMoeDecodeArgs c = a.c();
  detail::check(msq_moe_decode_static(e.stream, &c));
}
enum class MoePart { All, SharedGu, AfterSharedGu, Shared, Routed, SharedDown };  // reference: quant.hpp:85
inline void encode_moe_decode_table_part(Enc& e, const MoeDecodeArgs& a, const Buffer& table, MoePart part) {
  const MsqMoeDecodeArgs c = a.c();
  const MsqBuffer t = table.c();
  detail::check(msq_moe_decode_table_part(e.stream, &c, &t, (int)part));
}

struct MoePrefillArgs {  // reference: quant.hpp:93-116
  QType t_gate_up = QType::IQ1_S, t_down = QType::IQ1_S;
  int n_tokens = 0;
  int n_exp = 0;
  const ExpertSlot* slots = nullptr;
  const int* offs = nullptr;
  Buffer tok, wt, slot_of;
  int k_per_token = 6;
  bool has_shared = true;
  QType t_shared = QType::Q6_K;
  ExpertSlot shared;
  Buffer X, Y, scratch;
  int path = -1;
  int shared_dense = -1;
  int dim = kExpertDim, inter = kExpertInter;  // not in the reference
  bool x_is_bf16 = false;                      // not in the reference: activations given as bf16 instead of F32
};
inline size_t moe_prefill_scratch_bytes(int total_entries, int n_tokens, int n_exp = 384, int dim = kExpertDim,
                                        int inter = kExpertInter) {
  return msq_moe_prefill_scratch_bytes(total_entries, n_tokens, n_exp, dim, inter);
}
inline void encode_moe_prefill(Enc& e, const MoePrefillArgs& a) {
  std::vector<MsqExpertSlot> slots((size_t)(a.n_exp > 0 ? a.n_exp : 0));
  for (int j = 0; j < a.n_exp; j++) slots[(size_t)j] = a.slots[j].c();
  MsqMoePrefillArgs c{};
  c.t_gate_up = (int)a.t_gate_up; c.t_down = (int)a.t_down; c.n_tokens = a.n_tokens; c.n_exp = a.n_exp;
  c.slots = slots.data(); c.offs = a.offs; c.tok = a.tok.c(); c.wt = a.wt.c(); c.slot_of = a.slot_of.c();
  c.k_per_token = a.k_per_token; c.has_shared = a.has_shared; c.t_shared = (int)a.t_shared; c.shared = a.shared.c();
  c.X = a.X.c(); c.Y = a.Y.c(); c.scratch = a.scratch.c(); c.path = a.path; c.shared_dense = a.shared_dense;
  c.dim = a.dim; c.inter = a.inter; c.x_is_bf16 = a.x_is_bf16;
  detail::check(msq_moe_prefill(e.stream, &c));
}

}  // namespace q
}  // namespace ms
