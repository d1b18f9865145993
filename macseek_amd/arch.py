"""Host-side mirror of the reference's router operators (namespace ms::arch, src/kernels/arch.hpp:79-97) over the C ABI.

Only the part of that module which feeds the MoE kernels is here: top-6 selection from logits, the fused decode
router (F32 / BF16 matvec + selection in one launch) and the expert-sorted routing lists of the prefill grouped GEMM.
`encode_*` functions only enqueue work on the encoder's stream; errors raise QuantError. No CPU fallback.
"""
import ctypes as C

from . import _lib
from ._lib import MsqRouteLists
from .quant import Buffer, QType, _bp, _check

N_EXPERTS, TOP_K, ROUTE_SCALE = 384, 6, 1.5  # reference: src/kernels/arch_router.metal:5-6, arch.hpp:80


class Scratch:
    """reference: ms::arch::Scratch (router_logits + counter part only). Zeroed once at creation."""

    def __init__(self, n_exp=N_EXPERTS, device="cuda:0"):
        import torch
        self.n_exp = n_exp
        self.mem = torch.zeros(_lib.load().msq_router_scratch_bytes(n_exp), dtype=torch.uint8, device=device)
        self.router_logits = Buffer.of(self.mem).sub(0, n_exp * 4)

    @staticmethod
    def create(n_exp=N_EXPERTS, device="cuda:0"):
        return Scratch(n_exp, device)


def encode_router_topk(e, logits, bias, ids, w, n, n_exp=N_EXPERTS, route_scale=ROUTE_SCALE):  # reference: arch.hpp:84-85
    _check(_lib.load().msq_router_topk(e.handle, _bp(logits), _bp(bias), _bp(ids), _bp(w), n, n_exp, route_scale))


def encode_router_fused(e, x, W, bias, ids, w, s, dim, wtype=QType.F32, route_scale=ROUTE_SCALE):  # reference: arch.hpp:79-83
    _check(_lib.load().msq_router_fused(e.handle, int(wtype), _bp(x), _bp(W), _bp(bias), _bp(Buffer.of(s.mem)), _bp(ids),
                                        _bp(w), dim, s.n_exp, route_scale))


class RouteLists:
    """reference: ms::arch::RouteLists (arch.hpp:87-96)."""

    def __init__(self, max_tokens, n_exp=N_EXPERTS, device="cuda:0"):
        import torch
        self.max_tokens, self.n_exp = max_tokens, n_exp
        n = max(1, max_tokens * TOP_K)
        self.t_counts = torch.zeros(n_exp, dtype=torch.int32, device=device)
        self.t_offsets = torch.zeros(n_exp + 1, dtype=torch.int32, device=device)
        self.t_entry = torch.zeros(n, dtype=torch.int32, device=device)
        self.t_tok = torch.zeros(n, dtype=torch.int32, device=device)
        self.t_w = torch.zeros(n, dtype=torch.float32, device=device)
        self.t_slot_of = torch.zeros(n, dtype=torch.int32, device=device)
        self.counts, self.offsets, self.entry = Buffer.of(self.t_counts), Buffer.of(self.t_offsets), Buffer.of(self.t_entry)
        self.tok, self.w, self.slot_of = Buffer.of(self.t_tok), Buffer.of(self.t_w), Buffer.of(self.t_slot_of)

    @staticmethod
    def create(max_tokens, n_exp=N_EXPERTS, device="cuda:0"):
        return RouteLists(max_tokens, n_exp, device)

    def c(self):
        return MsqRouteLists(self.counts.c(), self.offsets.c(), self.entry.c(), self.tok.c(), self.w.c(), self.slot_of.c(),
                             self.max_tokens)


def encode_route_lists(e, ids, w, n, L):  # reference: arch.hpp:97
    _check(_lib.load().msq_route_lists(e.handle, _bp(ids), _bp(w), n, L.n_exp, C.byref(L.c())))


def encode_rmsnorm(e, x, w, y, rows, dim, eps, in_stride=0, out_stride=0):  # reference: arch.hpp:127-130
    _check(_lib.load().msq_rmsnorm(e.handle, _bp(x), _bp(w), _bp(y), rows, dim, eps, in_stride, out_stride))
