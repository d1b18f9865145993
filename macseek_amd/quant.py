"""Host-side mirror of the reference operator API (namespace ms::q, src/kernels/quant.hpp) over the C ABI.

Names, argument order and meaning follow the reference: `encode_*` functions only enqueue work on the encoder's
stream. Where the reference prints "macseek quant: ... unsupported" and aborts (src/kernels/quant.mm:34-37) these
functions raise QuantError with the same message. There is no CPU fallback: without libmsq.so every call raises.
"""
import ctypes as C
import enum

from . import _lib
from ._lib import MsqBuffer, MsqExpertSlot, MsqMoeDecodeArgs, MsqMoePrefillArgs, MsqMvCfg


class QType(enum.IntEnum):  # reference: src/kernels/quant_types.hpp:9-11 (ggml type ids)
    F32 = 0
    F16 = 1
    Q8_0 = 8
    Q5_K = 13
    Q6_K = 14
    IQ2_XXS = 16
    IQ1_S = 19
    IQ4_NL = 20
    BF16 = 30


class QuantError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(msg)
        self.code = code


def _check(rc):
    if rc != 0:
        raise QuantError(rc, _lib.load().msq_last_error().decode())


def block_elems(t):
    return _lib.load().msq_block_elems(int(t))


def block_bytes(t):
    return _lib.load().msq_block_bytes(int(t))


def row_bytes(t, cols):
    return _lib.load().msq_row_bytes(int(t), int(cols))


def type_name(t):
    return _lib.load().msq_type_name(int(t)).decode()


class Buffer:
    """reference: ms::Buffer (src/core/metal.hpp:11-18). A device allocation (kept alive through `owner`), a byte
    offset and the usable size from that offset."""

    __slots__ = ("dev", "off", "size", "owner")

    def __init__(self, dev=0, off=0, size=0, owner=None):
        self.dev, self.off, self.size, self.owner = int(dev), int(off), int(size), owner

    @staticmethod
    def of(tensor):
        """View of a whole torch tensor (must live on the GPU and be contiguous)."""
        assert tensor.is_contiguous()
        return Buffer(tensor.data_ptr(), 0, tensor.numel() * tensor.element_size(), tensor)

    def sub(self, o, s):
        assert o + s <= self.size
        return Buffer(self.dev, self.off + o, s, self.owner)

    def c(self):
        return MsqBuffer(self.dev, self.off, self.size)


class MvCfg:  # reference: ms::q::MvCfg (quant.hpp:12)
    def __init__(self, nr=0, rsg=0, ks=0):
        self.nr, self.rsg, self.ks = nr, rsg, ks


class Enc:
    """reference: ms::Enc (src/core/metal.hpp:37-71) reduced to what the quant operators need: a stream to enqueue
    on. barrier() is a no-op because a HIP stream is in-order; wait() blocks until the stream has drained."""

    def __init__(self, stream=None):
        import torch
        self._torch = torch
        self.stream = stream if stream is not None else torch.cuda.current_stream()

    @property
    def handle(self):
        return C.c_void_p(self.stream.cuda_stream)

    def barrier(self):
        pass

    def wait(self):
        self.stream.synchronize()


def _bp(b):
    return C.byref(b.c()) if b is not None else None


def matvec_supported(t):  # reference: quant.hpp:14
    return bool(_lib.load().msq_matvec_supported(int(t)))


def matvec_cfg(t, rows, cols):  # reference: quant.hpp:16-18
    out = MsqMvCfg()
    _check(_lib.load().msq_matvec_cfg(int(t), rows, cols, C.byref(out)))
    return MvCfg(out.nr, out.rsg, out.ks)


def encode_matvec(e, t, W, rows, cols, x, y, accumulate=False, groups=1, cfg=None):  # reference: quant.hpp:29-30
    c = MsqMvCfg(cfg.nr, cfg.rsg, cfg.ks) if cfg is not None else None
    _check(_lib.load().msq_matvec(e.handle, int(t), _bp(W), rows, cols, _bp(x), _bp(y), int(bool(accumulate)), groups,
                                  C.byref(c) if c is not None else None))


def encode_matvec_rmsnorm(e, t, W, rows, cols, x, norm_w, eps, y, tiles_per_tg=0):  # reference: quant.hpp:20-26
    _check(_lib.load().msq_matvec_rmsnorm(e.handle, int(t), _bp(W), rows, cols, _bp(x), _bp(norm_w), eps, _bp(y), tiles_per_tg))


def encode_matvec_n(e, t, W, rows, cols, X, Y, n, accumulate=False, groups=1):  # reference: quant.hpp:32-35
    _check(_lib.load().msq_matvec_n(e.handle, int(t), _bp(W), rows, cols, _bp(X), _bp(Y), n, int(bool(accumulate)), groups))


def encode_matmul(e, t, W, rows, cols, X, Y, n, accumulate=False):  # reference: quant.hpp:40-41
    _check(_lib.load().msq_matmul(e.handle, int(t), _bp(W), rows, cols, _bp(X), _bp(Y), n, int(bool(accumulate))))


def encode_f32_to_f16(e, X, X16, count):  # reference: quant.hpp:42
    _check(_lib.load().msq_f32_to_f16(e.handle, _bp(X), _bp(X16), count))


def encode_matmul_h(e, t, W, rows, cols, X16, Y, n, accumulate=False, x_stride=0):  # reference: quant.hpp:43-45
    _check(_lib.load().msq_matmul_h(e.handle, int(t), _bp(W), rows, cols, _bp(X16), _bp(Y), n, int(bool(accumulate)), x_stride))


def encode_dequant(e, t, W, n_elems, out):
    """Whole-buffer dequantization to fp32 (bit-exact with ref::dequant_row, tests/ref/dequant.cpp:34-120)."""
    _check(_lib.load().msq_dequant(e.handle, int(t), _bp(W), n_elems, _bp(out)))


# ---------------------------------------------------------------------------------------------- MoE, one token
kExpertDim, kExpertInter, kMaxRouted = 5120, 2304, 6  # reference: quant.hpp:49 (defaults of dim / inter here)


class ExpertSlot:  # reference: ms::q::ExpertSlot (quant.hpp:51-53)
    def __init__(self, gate=None, up=None, down=None):
        self.gate, self.up, self.down = gate or Buffer(), up or Buffer(), down or Buffer()

    def c(self):
        return MsqExpertSlot(self.gate.c(), self.up.c(), self.down.c())


class MoePart(enum.IntEnum):  # reference: ms::q::MoePart (quant.hpp:85)
    All = 0
    SharedGu = 1
    AfterSharedGu = 2
    Shared = 3
    Routed = 4
    SharedDown = 5
    Gu = 6      # no reference counterpart: the gate/up kernel of All alone
    Down = 7    # ... and its down kernel alone (Gu then Down == All, bit-identical)


class MoeDecodeArgs:
    """reference: ms::q::MoeDecodeArgs (quant.hpp:55-71) plus dim / inter (defaults = the reference constants)."""

    def __init__(self):
        self.t_gate_up = QType.IQ1_S
        self.t_down = QType.IQ1_S
        self.n_routed = 6
        self.slot = [ExpertSlot() for _ in range(kMaxRouted)]
        self.weights = Buffer()
        self.has_shared = True
        self.t_shared = QType.Q6_K
        self.shared = ExpertSlot()
        self.x = Buffer()
        self.y = Buffer()
        self.scratch = Buffer()
        self.gu_nr = self.gu_rsg = self.d_nr = self.d_rsg = 0
        self.dim, self.inter = kExpertDim, kExpertInter

    def c(self):
        a = MsqMoeDecodeArgs()
        a.t_gate_up, a.t_down, a.n_routed = int(self.t_gate_up), int(self.t_down), int(self.n_routed)
        for i in range(kMaxRouted):
            a.slot[i] = self.slot[i].c()
        a.weights = self.weights.c()
        a.has_shared, a.t_shared, a.shared = int(bool(self.has_shared)), int(self.t_shared), self.shared.c()
        a.x, a.y, a.scratch = self.x.c(), self.y.c(), self.scratch.c()
        a.gu_nr, a.gu_rsg, a.d_nr, a.d_rsg = self.gu_nr, self.gu_rsg, self.d_nr, self.d_rsg
        a.dim, a.inter = self.dim, self.inter
        return a


def moe_decode_scratch_bytes(inter=kExpertInter):  # reference: quant.hpp:72
    return _lib.load().msq_moe_decode_scratch_bytes(inter)


def encode_moe_decode(e, a):  # reference: quant.hpp:73-75
    _check(_lib.load().msq_moe_decode(e.handle, C.byref(a.c())))


def encode_moe_decode_table(e, a, table):  # reference: quant.hpp:76-78
    _check(_lib.load().msq_moe_decode_table(e.handle, C.byref(a.c()), _bp(table)))


def encode_moe_decode_table_part(e, a, table, part):  # reference: quant.hpp:79-86
    _check(_lib.load().msq_moe_decode_table_part(e.handle, C.byref(a.c()), _bp(table), int(part)))


def encode_moe_decode_static(e, a):
    """encode_moe_decode without caller scratch (no reference counterpart): h lives in the library's static device
    array, nothing is allocated; a.scratch is ignored. inter <= moe_decode_static_max_inter()."""
    _check(_lib.load().msq_moe_decode_static(e.handle, C.byref(a.c())))


def moe_decode_static_max_inter():
    return _lib.load().msq_moe_decode_static_max_inter()


# ---------------------------------------------------------------------------------------------- MoE, prefill
class MoePrefillArgs:
    """reference: ms::q::MoePrefillArgs (quant.hpp:93-116) plus dim / inter / x_is_bf16. `slots` is a list of
    ExpertSlot (host), `offs` a list of n_exp + 1 ints (host); tok / wt / slot_of / X / Y / scratch are device Buffers."""

    def __init__(self):
        self.t_gate_up = QType.IQ1_S
        self.t_down = QType.IQ1_S
        self.n_tokens = 0
        self.n_exp = 0
        self.slots = []
        self.offs = [0]
        self.tok = Buffer()
        self.wt = Buffer()
        self.slot_of = Buffer()
        self.k_per_token = 6
        self.has_shared = True
        self.t_shared = QType.Q6_K
        self.shared = ExpertSlot()
        self.X = Buffer()
        self.Y = Buffer()
        self.scratch = Buffer()
        self.path = -1
        self.shared_dense = -1
        self.dim, self.inter = kExpertDim, kExpertInter
        self.x_is_bf16 = False

    def c(self):
        a = MsqMoePrefillArgs()
        a.t_gate_up, a.t_down, a.n_tokens, a.n_exp = int(self.t_gate_up), int(self.t_down), self.n_tokens, self.n_exp
        self._slots = (MsqExpertSlot * max(1, self.n_exp))(*[s.c() for s in self.slots[:self.n_exp]])
        self._offs = (C.c_int * (self.n_exp + 1))(*self.offs[:self.n_exp + 1])
        a.slots, a.offs = self._slots, self._offs
        a.tok, a.wt, a.slot_of = self.tok.c(), self.wt.c(), self.slot_of.c()
        a.k_per_token, a.has_shared, a.t_shared, a.shared = self.k_per_token, int(bool(self.has_shared)), int(self.t_shared), self.shared.c()
        a.X, a.Y, a.scratch = self.X.c(), self.Y.c(), self.scratch.c()
        a.path, a.shared_dense, a.dim, a.inter, a.x_is_bf16 = self.path, self.shared_dense, self.dim, self.inter, int(bool(self.x_is_bf16))
        return a


def moe_prefill_scratch_bytes(total_entries, n_tokens, n_exp=384, dim=kExpertDim, inter=kExpertInter):  # reference: quant.hpp:117
    return _lib.load().msq_moe_prefill_scratch_bytes(total_entries, n_tokens, n_exp, dim, inter)


def encode_moe_prefill(e, a):  # reference: quant.hpp:118
    _check(_lib.load().msq_moe_prefill(e.handle, C.byref(a.c())))
