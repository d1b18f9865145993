"""GGUF reader tests (CPU: the parser is host code inside libmsq.so; nothing here touches a GPU).

Mirrors the reference's tests/test_gguf.cpp -- type table, split expansion, tensor table (name, type, dims, nbytes,
split, absolute offset), typed metadata incl. arrays -- on files written by tests/gguf_writer.py, because the real model
the reference parses is not available. The reference's docs/tensors.txt rows are checked for what they pin without the
file: nbytes of every listed tensor from its type and dims.
"""
import os

import numpy as np
import pytest

import gguf_writer as W
import oracle as O
from macseek_amd import gguf, quant as q


def test_type_table_and_split_expansion():  # tests/test_gguf.cpp:24-29
    assert gguf.type_bytes(19, 256) == 50 and gguf.type_bytes(16, 256) == 66 and gguf.type_bytes(20, 256) == 144
    assert gguf.type_bytes(14, 5120) == 4200 and gguf.type_bytes(39, 32) == 17 and gguf.type_bytes(99, 256) == 0
    assert gguf.type_name(19) == "IQ1_S" and gguf.type_name(30) == "BF16" and gguf.type_name(99) == "?"
    for t in (0, 1, 8, 13, 14, 16, 19, 20, 30):  # the kernels' own geometry agrees
        assert gguf.type_bytes(t, 512) == q.row_bytes(q.QType(t), 512)
    assert gguf.expand_splits_count("/a/b-00002-of-00005.gguf") == 5 and gguf.expand_splits_count("/a/b.gguf") == 1
    assert gguf.expand_splits_count("/a/b-0002-of-00005.gguf") == 1


# rows of the reference's docs/tensors.txt (name, type, dims, nbytes): nbytes follows from type and dims
DOC_ROWS = [("blk.0.attn_q_b.weight", 14, [1280, 32768], 34406400), ("blk.0.ffn_down_exps.weight", 19, [2304, 5120, 384], 884736000),
            ("blk.0.ffn_down_shexp.weight", 14, [2304, 5120], 9676800), ("blk.0.ffn_gate_inp.weight", 0, [5120, 384], 7864320),
            ("blk.0.attn_sinks.weight", 0, [64], 256)]


def test_nbytes_of_documented_tensors():
    for name, t, ne, nbytes in DOC_ROWS:
        assert gguf.type_bytes(t, int(np.prod(ne))) == nbytes, name


def make_model(tmp_path, align=32, version=3):
    rng = np.random.default_rng(7)
    kvs = [("general.architecture", W.STR, "deepseek41"), ("deepseek41.block_count", W.U32, 2),
           ("deepseek41.expert_count", W.U32, 4), ("deepseek41.expert_weights_norm", W.BOOL, 1),
           ("deepseek41.expert_weights_scale", W.F32, 1.5), ("neg", W.I16, -7), ("big", W.U64, 2 ** 63 + 5), ("dbl", W.F64, 0.1),
           ("tokenizer.ggml.tokens", W.ARR, (W.STR, ["<s>", "hello", "wor ld", ""])),
           ("deepseek41.ple.layer_multipliers", W.ARR, (W.I64, [76632096046245, -3, 82619226485591])),
           ("deepseek41.swiglu_clamp_exp", W.ARR, (W.F32, [10.0, 0.5])), ("empty", W.ARR, (W.I32, [])),
           ("nested", W.ARR, (W.ARR, [(W.I32, [1, 2, 3]), (W.I32, []), (W.I32, [-9])])), ("split.count", W.U16, 1)]
    tensors = []
    for name, t, ne in (("token_embd.weight", 30, [64, 10]), ("blk.0.attn_q_a.weight", 14, [256, 3]),
                        ("blk.0.ffn_gate_exps.weight", 19, [256, 8, 4]), ("odd", 24, [7]), ("blk.0.norm.weight", 0, [5])):
        tensors.append((name, t, ne, rng.integers(0, 256, gguf.type_bytes(t, int(np.prod(ne))), dtype=np.uint8)))
    path = str(tmp_path / "m.gguf")
    offs, data_off = W.write_gguf(path, kvs, tensors, alignment=align, version=version)
    return path, kvs, tensors, offs, data_off


@pytest.mark.parametrize("align,version", [(32, 3), (64, 3), (32, 2), (4096, 3)])
def test_parse_tensor_table_and_metadata(tmp_path, align, version):
    path, kvs, tensors, offs, data_off = make_model(tmp_path, align, version)
    g = gguf.Gguf(path)
    assert g.n_splits() == 1 and g.version() == version and g.alignment() == align and g.data_offset(0) == data_off
    assert g.path(0) == path
    got = g.tensors()
    assert [t.name for t in got] == [t[0] for t in tensors]  # file order
    for ti, (name, t, ne, data) in zip(got, tensors):
        assert ti.type == t and ti.n_dims == len(ne) and ti.ne[:len(ne)] == ne and ti.ne[len(ne):] == [1] * (4 - len(ne))
        assert ti.nbytes == data.size and ti.split == 0 and ti.offset == offs[name] and ti.offset % align == 0
        assert np.array_equal(g.read(ti), data)
        assert np.array_equal(g.read(ti, 1, data.size - 1), data[1:])
    assert g.find("blk.0.attn_q_a.weight").row_bytes() == 210 and g.find("nope") is None
    # metadata: typed scalars, strings, arrays, nested arrays; insertion order
    want_keys = [k for k, _, _ in kvs] + (["general.alignment"] if align != 32 else [])
    assert g.keys() == want_keys
    assert g.get_str("general.architecture") == "deepseek41" and g.get_i64("deepseek41.block_count") == 2
    assert g.kv_type("deepseek41.expert_weights_norm") == ("bool", None) and g.get_i64("deepseek41.expert_weights_norm") == 1
    assert g.get_f64("deepseek41.expert_weights_scale") == 1.5 and g.get_i64("deepseek41.expert_weights_scale") == 1
    assert g.get_i64("neg") == -7 and g.get_f64("neg") == -7.0 and g.get_f64("dbl") == 0.1
    assert g.get_i64("big") & (2 ** 64 - 1) == 2 ** 63 + 5
    assert g.get_arr_str("tokenizer.ggml.tokens") == ["<s>", "hello", "wor ld", ""]
    assert g.get_arr_i64("deepseek41.ple.layer_multipliers").tolist() == [76632096046245, -3, 82619226485591]
    assert g.get_arr_f32("deepseek41.swiglu_clamp_exp").tolist() == [10.0, 0.5]
    assert g.arr_len("empty") == 0 and g.kv_type("empty") == ("arr", "i32") and g.kv_type("nested") == ("arr", "arr")
    assert [v.tolist() for v in g.get_arr_nested_i64("nested")] == [[1, 2, 3], [], [-9]]
    # missing keys and mismatched kinds give the defaults (gguf.hpp:66-71)
    assert g.get_i64("missing", 42) == 42 and g.get_str("missing", "d") == "d" and g.get_i64("general.architecture", 3) == 3
    assert g.kv_type("missing") is None and g.arr_len("neg") == -1 and g.get_arr_str("missing") == []
    g.close()


def test_splits_are_merged(tmp_path):
    rng = np.random.default_rng(1)
    d1, d2 = rng.integers(0, 256, 34 * 4, dtype=np.uint8), rng.integers(0, 256, 50 * 2, dtype=np.uint8)
    p1, p2 = str(tmp_path / "x-00001-of-00002.gguf"), str(tmp_path / "x-00002-of-00002.gguf")
    o1, _ = W.write_gguf(p1, [("general.architecture", W.STR, "a"), ("split.count", W.U16, 2), ("only1", W.I32, 1)], [("t1", 8, [32, 4], d1)])
    o2, _ = W.write_gguf(p2, [("general.architecture", W.STR, "b"), ("only2", W.I32, 2)], [("t2", 19, [256, 2], d2)])
    for start in (p1, p2):  # either split names the whole set
        g = gguf.Gguf(start)
        assert g.n_splits() == 2 and [os.path.basename(g.path(i)) for i in range(2)] == [os.path.basename(p1), os.path.basename(p2)]
        assert g.get_str("general.architecture") == "a" and g.get_i64("only1") == 1 and g.get_i64("only2") == 2  # first wins
        t1, t2 = g.find("t1"), g.find("t2")
        assert (t1.split, t1.offset, t2.split, t2.offset) == (0, o1["t1"], 1, o2["t2"])
        assert np.array_equal(g.read(t1), d1) and np.array_equal(g.read(t2), d2)
        g.close()


def test_bad_files_are_rejected(tmp_path):
    p = str(tmp_path / "bad.gguf")
    with pytest.raises(q.QuantError, match="cannot open"):
        gguf.Gguf(p)
    open(p, "wb").write(b"GGML" + b"\0" * 64)
    with pytest.raises(q.QuantError, match="not a GGUF file"):
        gguf.Gguf(p)
    path, *_ = make_model(tmp_path)
    raw = open(path, "rb").read()
    open(p, "wb").write(raw[:4] + (7).to_bytes(4, "little") + raw[8:])
    with pytest.raises(q.QuantError, match="unsupported GGUF version 7"):
        gguf.Gguf(p)
    open(p, "wb").write(raw[:200])
    with pytest.raises(q.QuantError, match="bad metadata|truncated|bad tensor table"):
        gguf.Gguf(p)
    open(p, "wb").write(raw[:-40])  # the last tensor's data is cut short
    with pytest.raises(q.QuantError, match="runs past the end of the file"):
        gguf.Gguf(p)
    # a row that is not a whole number of blocks
    W.write_gguf(p, [], [("r", 14, [100, 2], np.zeros(10, np.uint8))])
    with pytest.raises(q.QuantError, match="ragged row"):
        gguf.Gguf(p)
    # an alignment that is no power of two; dimensions whose product does not fit 64 bits
    W.write_gguf(p, [], [("r", 0, [4], np.zeros(16, np.uint8))], alignment=24)
    with pytest.raises(q.QuantError, match="general.alignment is not a power of two"):
        gguf.Gguf(p)
    W.write_gguf(p, [], [("r", 0, [1 << 40, 1 << 40], np.zeros(16, np.uint8))])
    with pytest.raises(q.QuantError, match="product overflows"):
        gguf.Gguf(p)


def test_expert_layout(tmp_path):  # src/store/experts.mm:36-56
    E, dim, inter = 4, 512, 256
    tensors = []
    for layer in range(2):
        for nm, t, ne in (("ffn_gate_exps", 19, [dim, inter, E]), ("ffn_up_exps", 19, [dim, inter, E]), ("ffn_down_exps", 16, [inter, dim, E])):
            tensors.append(("blk.%d.%s.weight" % (layer, nm), t, ne, O.random_blocks(t, dim * inter * E, 5 + layer)))
    path = str(tmp_path / "e.gguf")
    W.write_gguf(path, [("general.architecture", W.STR, "deepseek41")], tensors)
    g = gguf.Gguf(path)
    L = g.expert_layout(1)
    assert L.n_experts == E and list(L.type) == [19, 19, 16] and list(L.rows) == [inter, inter, dim] and list(L.cols) == [dim, dim, inter]
    assert list(L.stride) == [inter * 100, inter * 100, dim * 66] and [g.tensor(i).name for i in L.tensor] == [t[0] for t in tensors[3:]]
    assert L.arena_bytes == E * sum((s + 255) // 256 * 256 for s in L.stride)
    with pytest.raises(q.QuantError, match=r"tensor blk\.2\.ffn_gate_exps\.weight is missing"):
        g.expert_layout(2)
