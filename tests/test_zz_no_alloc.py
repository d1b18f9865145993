"""The allocation-free one-token MoE entry point (msq_moe_decode_static: h rows in the library's static device array)
against msq_moe_decode with caller scratch, through the C ABI: bit-identical y on two calls in a row, the second with a
smaller layer, and the size limit is refused with a clear message."""
import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import quant as q
from test_moe_decode_gpu import SMALL_SHAPE_CHAIN_TOL, Layer
from util import up

pytestmark = pytest.mark.gpu


def run_both(L):
    e = q.Enc()
    y_ref = up(L.y0.copy())
    q.encode_moe_decode(e, L.args(y_ref))
    e.wait()
    y_static = up(L.y0.copy())
    a = L.args(y_static)
    a.scratch = q.Buffer()  # ignored by the static entry point
    q.encode_moe_decode_static(e, a)
    e.wait()
    return y_ref, y_static


def test_static_scratch_entry_point_matches_caller_scratch(dev):
    big = Layer(O.IQ1_S, O.IQ1_S, O.IQ2_XXS, 6, True, 7168, 2048)
    y_ref, y_static = run_both(big)
    assert torch.equal(y_ref, y_static)
    big.check(y_static, None, "static scratch, 7168/2048")
    # second call, smaller layer: the array still holds the first call's h rows beyond the new layer's
    small = Layer(O.IQ1_S, O.IQ2_XXS, O.Q8_0, 2, True, 512, 256, seed=300)
    y_ref, y_static = run_both(small)
    assert torch.equal(y_ref, y_static)
    small.check(y_static, None, "static scratch, 512/256", chain_tol=SMALL_SHAPE_CHAIN_TOL)
    # and the first shape again
    y_ref, y_static = run_both(big)
    assert torch.equal(y_ref, y_static)


def test_static_entry_point_allocates_nothing_and_can_be_captured(dev):
    """What the entry point exists for: a call enqueues and allocates nothing, so it can sit inside a HIP graph. After
    one warm-up call (the first call on a device looks the array's address up and sets the kernels' LDS limits) the
    device's free memory is the same before and after a call, and a graph that holds the call repeats the eager result
    bit for bit on every replay, with eager work and synchronizations between the replays."""
    L = Layer(O.IQ1_S, O.IQ1_S, O.IQ2_XXS, 6, True, 7168, 2048)
    y0 = up(L.y0.copy())
    y_eager, y_graph = up(L.y0.copy()), up(L.y0.copy())
    e = q.Enc()

    def static_args(y):
        a = L.args(y)
        a.scratch = q.Buffer()
        return a

    q.encode_moe_decode_static(e, static_args(y_eager))  # warm-up
    e.wait()
    y_eager.copy_(y0)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    q.encode_moe_decode_static(e, static_args(y_eager))
    e.wait()
    assert torch.cuda.mem_get_info()[0] == free_before
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        q.encode_moe_decode_static(q.Enc(torch.cuda.current_stream()), static_args(y_graph))
    for rep in range(4):
        y_graph.copy_(y0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_eager), f"replay {rep} differs from the eager result"
        _ = (y0 * 2).sum().item()  # eager work between the replays


def test_static_scratch_limit(dev):
    assert q.moe_decode_static_max_inter() == 4096
    L = Layer(O.IQ2_XXS, O.IQ1_S, O.IQ2_XXS, 1, True, 256, 8192)
    y = up(L.y0.copy())
    a = L.args(y)
    with pytest.raises(q.QuantError, match="exceeds the static scratch limit of 4096"):
        q.encode_moe_decode_static(q.Enc(), a)
    assert np.array_equal(y.cpu().numpy(), L.y0)
