// C++20 shim: the router part of the reference's ms::arch operator API (src/kernels/arch.hpp:79-97) over the libmsq C
// ABI -- top-6 selection from logits, the fused decode router and the expert-sorted routing lists that feed
// ms::q::encode_moe_decode* and ms::q::encode_moe_prefill. Same names and argument order; what differs is spelled out
// per function. Misuse prints the library's message and aborts, as the reference does.
#pragma once
#include "quant.hpp"

namespace ms::arch {

constexpr int kExperts = 384, kTopK = MSQ_MAX_ROUTED;  // reference: src/kernels/arch_router.metal:5-6
constexpr float kRouteScale = 1.5f;                    // reference: arch_router.metal:53

// reference: ms::arch::Scratch (its router_logits + counter members). `mem` is device memory of at least
// msq_router_scratch_bytes(n_exp) bytes that the caller zeroed once; router_logits views its first n_exp floats.
struct Scratch {
  Buffer mem;
  int n_exp = kExperts;
  Buffer router_logits() const { return mem.sub(0, (size_t)n_exp * 4); }
};

// reference: arch.hpp:79-83. W is [n_exp][dim] F32 (wtype defaults to it) or BF16; dim is explicit (the reference
// hard-codes 5120).
inline void encode_router_fused(Enc& e, Buffer x, Buffer W, Buffer bias, Buffer ids, Buffer w, const Scratch& s, int dim,
                                q::QType wtype = q::QType::F32, float route_scale = kRouteScale) {
  const MsqBuffer xb = x.c(), wb = W.c(), bb = bias.c(), sb = s.mem.c(), ib = ids.c(), ob = w.c();
  q::detail::check(msq_router_fused(e.stream, (int)wtype, &xb, &wb, &bb, &sb, &ib, &ob, dim, s.n_exp, route_scale));
}

// reference: arch.hpp:84-85
inline void encode_router_topk(Enc& e, Buffer logits, Buffer bias, Buffer ids, Buffer w, int n, int n_exp = kExperts,
                               float route_scale = kRouteScale) {
  const MsqBuffer lb = logits.c(), bb = bias.c(), ib = ids.c(), ob = w.c();
  q::detail::check(msq_router_topk(e.stream, &lb, &bb, &ib, &ob, n, n_exp, route_scale));
}

// reference: arch.hpp:87-96. The buffers are caller-allocated device memory here (the reference's create() allocates
// them from its Metal device): counts u32[n_exp], offsets u32[n_exp + 1], entry / tok / slot_of u32[6 max_tokens],
// w f32[6 max_tokens].
struct RouteLists {
  Buffer counts, offsets, entry, tok, w, slot_of;
  int max_tokens = 0;
  int n_exp = kExperts;
  MsqRouteLists c() const { return MsqRouteLists{counts.c(), offsets.c(), entry.c(), tok.c(), w.c(), slot_of.c(), max_tokens}; }
};

// reference: arch.hpp:97
inline void encode_route_lists(Enc& e, Buffer ids, Buffer w, int n, const RouteLists& L) {
  const MsqBuffer ib = ids.c(), wb = w.c();
  const MsqRouteLists l = L.c();
  q::detail::check(msq_route_lists(e.stream, &ib, &wb, n, L.n_exp, &l));
}

// reference: arch.hpp:127-130 (w.buf == nullptr: no weight)
inline void encode_rmsnorm(Enc& e, Buffer x, Buffer w, Buffer y, int rows, int dim, float eps, int in_stride = 0,
                           int out_stride = 0) {
  const MsqBuffer xb = x.c(), wb = w.c(), yb = y.c();
  q::detail::check(msq_rmsnorm(e.stream, &xb, w.buf ? &wb : nullptr, &yb, rows, dim, eps, in_stride, out_stride));
}

}  // namespace ms::arch
