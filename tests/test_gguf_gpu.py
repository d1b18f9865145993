"""GPU side of the GGUF reader: tensors loaded into device memory, a layer's experts placed in HBM at 256-byte
aligned offsets, and the placed experts run through msq_moe_decode against the oracle fed with the file's bytes."""
import numpy as np
import pytest
import torch

import gguf_writer as W
import oracle as O
from macseek_amd import gguf, quant as q
from util import up

pytestmark = pytest.mark.gpu


def test_place_experts_bytes_and_alignment(dev, tmp_path):
    E = 5
    tensors = []
    for nm, t, ne in (("ffn_gate_exps", 19, [256, 8, E]), ("ffn_up_exps", 16, [512, 3, E]), ("ffn_down_exps", 19, [256, 64, E])):
        tensors.append(("blk.3.%s.weight" % nm, t, ne, O.random_blocks(t, int(np.prod(ne)), 40 + len(tensors))))
    tensors.append(("blk.3.ffn_gate_shexp.weight", 14, [256, 6], O.random_blocks(14, 256 * 6, 50)))
    path = str(tmp_path / "p.gguf")
    W.write_gguf(path, [("general.architecture", W.STR, "deepseek41")], tensors)
    g = gguf.Gguf(path)
    L = g.expert_layout(3)
    assert list(L.stride) == [400, 396, 3200]  # 400 and 396 are padded to 512, 3200 to 3328
    assert L.arena_bytes == E * (512 + 512 + 3328)
    arena = torch.full((L.arena_bytes + 256,), 0xEE, dtype=torch.uint8, device=dev)
    e = q.Enc()
    L2, slots = g.place_experts(e, 3, q.Buffer.of(arena).sub(0, L.arena_bytes))
    e.wait()
    host = arena.cpu().numpy()
    base = arena.data_ptr()
    for ex in range(E):
        for k, b in enumerate((slots[ex].gate, slots[ex].up, slots[ex].down)):
            off = b.dev + b.off - base
            assert off % 256 == 0 and b.size == L.stride[k]
            want = tensors[k][3][ex * L.stride[k]:(ex + 1) * L.stride[k]]
            assert np.array_equal(host[off:off + b.size], want), (ex, k)
    assert (host[L.arena_bytes:] == 0xEE).all()
    # a plain tensor (the shared expert's gate) and a sub-range of it
    t = g.find("blk.3.ffn_gate_shexp.weight")
    dst = torch.zeros(t.nbytes + 16, dtype=torch.uint8, device=dev)
    g.load_tensor(e, t, q.Buffer.of(dst).sub(0, t.nbytes))
    e.wait()
    assert np.array_equal(dst.cpu().numpy()[:t.nbytes], tensors[3][3]) and not dst[t.nbytes:].any()
    g.load_tensor(e, t, q.Buffer.of(dst).sub(0, 210), byte_off=420, length=210)
    e.wait()
    assert np.array_equal(dst.cpu().numpy()[:210], tensors[3][3][420:630])
    with pytest.raises(q.QuantError, match="arena missing, smaller than"):
        g.place_experts(e, 3, q.Buffer.of(arena).sub(0, L.arena_bytes - 256))
    with pytest.raises(q.QuantError, match="bad tensor index or range"):
        g.load_tensor(e, t, q.Buffer.of(dst), byte_off=t.nbytes, length=1)


def test_placed_experts_run_the_moe_layer(dev, tmp_path):
    E, dim, inter = 8, 512, 256
    G = O.random_blocks(O.IQ1_S, dim * inter * E, 1)
    U = O.random_blocks(O.IQ1_S, dim * inter * E, 2)
    D = O.random_blocks(O.IQ2_XXS, dim * inter * E, 3)
    SG, SU, SD = (O.random_blocks(O.Q6_K, dim * inter, 4 + i) for i in range(3))
    path = str(tmp_path / "l.gguf")
    W.write_gguf(path, [("general.architecture", W.STR, "deepseek41"), ("deepseek41.expert_count", W.U32, E)],
                 [("blk.0.ffn_gate_exps.weight", 19, [dim, inter, E], G), ("blk.0.ffn_up_exps.weight", 19, [dim, inter, E], U),
                  ("blk.0.ffn_down_exps.weight", 16, [inter, dim, E], D), ("blk.0.ffn_gate_shexp.weight", 14, [dim, inter], SG),
                  ("blk.0.ffn_up_shexp.weight", 14, [dim, inter], SU), ("blk.0.ffn_down_shexp.weight", 14, [inter, dim], SD)])
    g = gguf.Gguf(path)
    assert g.get_i64("deepseek41.expert_count") == E
    e = q.Enc()
    L = g.expert_layout(0)
    arena = torch.zeros(L.arena_bytes, dtype=torch.uint8, device=dev)
    _, slots = g.place_experts(e, 0, q.Buffer.of(arena))
    shared = []
    for nm in ("gate", "up", "down"):
        t = g.find("blk.0.ffn_%s_shexp.weight" % nm)
        d = torch.zeros(t.nbytes, dtype=torch.uint8, device=dev)
        g.load_tensor(e, t, q.Buffer.of(d))
        shared.append(d)
    ids = [6, 1, 7, 0, 3, 5]
    w = np.array([0.31, 0.22, 0.17, 0.12, 0.1, 0.08], dtype=np.float32)
    x, y0 = O.randn(dim, 77), O.randn(dim, 78)
    a = q.MoeDecodeArgs()
    a.t_gate_up, a.t_down, a.t_shared, a.n_routed, a.has_shared = q.QType.IQ1_S, q.QType.IQ2_XXS, q.QType.Q6_K, 6, True
    for k, ex in enumerate(ids):
        gb, ub, db = gguf.slot_buffers(slots[ex], arena)
        a.slot[k] = q.ExpertSlot(gb, ub, db)
    a.shared = q.ExpertSlot(*[q.Buffer.of(d) for d in shared])
    wd, xd, yd = up(w), up(x), up(y0.copy())
    scratch = torch.zeros(q.moe_decode_scratch_bytes(inter) // 4, dtype=torch.float32, device=dev)
    a.weights, a.x, a.y, a.scratch, a.dim, a.inter = q.Buffer.of(wd), q.Buffer.of(xd), q.Buffer.of(yd), q.Buffer.of(scratch), dim, inter
    q.encode_moe_decode(e, a)
    e.wait()
    sg, sd = inter * 100, dim * 66  # per-expert slabs in the file
    Gs = [G[i * sg:(i + 1) * sg] for i in ids] + [SG]
    Us = [U[i * sg:(i + 1) * sg] for i in ids] + [SU]
    Ds = [D[i * sd:(i + 1) * sd] for i in ids] + [SD]
    ry, ymag, _, _ = O.moe_decode(O.IQ1_S, O.IQ2_XXS, O.Q6_K, 6, True, dim, inter, Gs, Us, Ds, w, x, y0)
    err = float(np.max(np.abs(yd.cpu().numpy() - ry) / (ymag + 1e-12)))
    print(f"  MoE layer on experts placed from a GGUF file: chain error {err:.2e}")
    assert err <= 1.5e-4  # whole chain on the smallest layer shape, 512-column rows and 256-column h rows (measured 8.7e-5)
