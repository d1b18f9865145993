"""ctypes binding of libmsq.so (the C ABI declared in include/msq.h). Fails loudly when the library is absent."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "libmsq.so")


class MsqBuffer(C.Structure):
    _fields_ = [("dev", C.c_void_p), ("off", C.c_size_t), ("size", C.c_size_t)]


class MsqMvCfg(C.Structure):
    _fields_ = [("nr", C.c_int), ("rsg", C.c_int), ("ks", C.c_int)]


class MsqExpertSlot(C.Structure):
    _fields_ = [("gate", MsqBuffer), ("up", MsqBuffer), ("down", MsqBuffer)]


MSQ_MAX_ROUTED = 6


class MsqMoeDecodeArgs(C.Structure):
    _fields_ = [("t_gate_up", C.c_int), ("t_down", C.c_int), ("n_routed", C.c_int),
                ("slot", MsqExpertSlot * MSQ_MAX_ROUTED), ("weights", MsqBuffer), ("has_shared", C.c_int),
                ("t_shared", C.c_int), ("shared", MsqExpertSlot), ("x", MsqBuffer), ("y", MsqBuffer),
                ("scratch", MsqBuffer), ("gu_nr", C.c_int), ("gu_rsg", C.c_int), ("d_nr", C.c_int), ("d_rsg", C.c_int),
                ("dim", C.c_int), ("inter", C.c_int)]


class MsqMoePrefillArgs(C.Structure):
    _fields_ = [("t_gate_up", C.c_int), ("t_down", C.c_int), ("n_tokens", C.c_int), ("n_exp", C.c_int),
                ("slots", C.POINTER(MsqExpertSlot)), ("offs", C.POINTER(C.c_int)), ("tok", MsqBuffer), ("wt", MsqBuffer),
                ("slot_of", MsqBuffer), ("k_per_token", C.c_int), ("has_shared", C.c_int), ("t_shared", C.c_int),
                ("shared", MsqExpertSlot), ("X", MsqBuffer), ("Y", MsqBuffer), ("scratch", MsqBuffer),
                ("path", C.c_int), ("shared_dense", C.c_int), ("dim", C.c_int), ("inter", C.c_int),
                ("x_is_bf16", C.c_int)]


class MsqRouteLists(C.Structure):
    _fields_ = [("counts", MsqBuffer), ("offsets", MsqBuffer), ("entry", MsqBuffer), ("tok", MsqBuffer),
                ("w", MsqBuffer), ("slot_of", MsqBuffer), ("max_tokens", C.c_int)]


class MsqGgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("type", C.c_int), ("n_dims", C.c_int), ("ne", C.c_int64 * 4), ("nbytes", C.c_uint64),
                ("split", C.c_int), ("offset", C.c_uint64)]


class MsqExpertLayout(C.Structure):
    _fields_ = [("n_experts", C.c_int), ("type", C.c_int * 3), ("rows", C.c_int64 * 3), ("cols", C.c_int64 * 3),
                ("stride", C.c_uint64 * 3), ("tensor", C.c_int * 3), ("arena_bytes", C.c_uint64)]


_lib = None

# name -> (restype, argtypes); every symbol include/msq.h declares
_BP = C.POINTER(MsqBuffer)
SIGNATURES = {
    "msq_init": (C.c_int, []),
    "msq_last_error": (C.c_char_p, []),
    "msq_device_ok": (C.c_int, []),
    "msq_block_elems": (C.c_int, [C.c_int]),
    "msq_block_bytes": (C.c_size_t, [C.c_int]),
    "msq_row_bytes": (C.c_size_t, [C.c_int, C.c_int64]),
    "msq_type_name": (C.c_char_p, [C.c_int]),
    "msq_matvec_supported": (C.c_int, [C.c_int]),
    "msq_matvec_cfg": (C.c_int, [C.c_int, C.c_int, C.c_int, C.POINTER(MsqMvCfg)]),
    "msq_matvec": (C.c_int, [C.c_void_p, C.c_int, _BP, C.c_int, C.c_int, _BP, _BP, C.c_int, C.c_int, C.POINTER(MsqMvCfg)]),
    "msq_matvec_rmsnorm": (C.c_int, [C.c_void_p, C.c_int, _BP, C.c_int, C.c_int, _BP, _BP, C.c_float, _BP, C.c_int]),
    "msq_rmsnorm": (C.c_int, [C.c_void_p, _BP, _BP, _BP, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int]),
    "msq_matvec_n": (C.c_int, [C.c_void_p, C.c_int, _BP, C.c_int, C.c_int, _BP, _BP, C.c_int, C.c_int, C.c_int]),
    "msq_f32_to_f16": (C.c_int, [C.c_void_p, _BP, _BP, C.c_size_t]),
    "msq_matmul_h": (C.c_int, [C.c_void_p, C.c_int, _BP, C.c_int, C.c_int, _BP, _BP, C.c_int, C.c_int, C.c_int]),
    "msq_matmul": (C.c_int, [C.c_void_p, C.c_int, _BP, C.c_int, C.c_int, _BP, _BP, C.c_int, C.c_int]),
    "msq_dequant": (C.c_int, [C.c_void_p, C.c_int, _BP, C.c_int64, _BP]),
    "msq_bw_probe": (C.c_int, [C.c_void_p, _BP, C.c_size_t, _BP]),
    "msq_moe_decode_scratch_bytes": (C.c_size_t, [C.c_int]),
    "msq_moe_decode": (C.c_int, [C.c_void_p, C.POINTER(MsqMoeDecodeArgs)]),
    "msq_moe_decode_table": (C.c_int, [C.c_void_p, C.POINTER(MsqMoeDecodeArgs), _BP]),
    "msq_moe_decode_table_part": (C.c_int, [C.c_void_p, C.POINTER(MsqMoeDecodeArgs), _BP, C.c_int]),
    "msq_moe_decode_static": (C.c_int, [C.c_void_p, C.POINTER(MsqMoeDecodeArgs)]),
    "msq_moe_decode_static_max_inter": (C.c_int, []),
    "msq_moe_prefill_scratch_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "msq_moe_prefill": (C.c_int, [C.c_void_p, C.POINTER(MsqMoePrefillArgs)]),
    "msq_router_topk": (C.c_int, [C.c_void_p, _BP, _BP, _BP, _BP, C.c_int, C.c_int, C.c_float]),
    "msq_router_scratch_bytes": (C.c_size_t, [C.c_int]),
    "msq_router_fused": (C.c_int, [C.c_void_p, C.c_int, _BP, _BP, _BP, _BP, _BP, _BP, C.c_int, C.c_int, C.c_float]),
    "msq_gguf_open": (C.c_int, [C.c_char_p, C.POINTER(C.c_void_p)]),
    "msq_gguf_close": (None, [C.c_void_p]),
    "msq_gguf_n_splits": (C.c_int, [C.c_void_p]),
    "msq_gguf_n_tensors": (C.c_int, [C.c_void_p]),
    "msq_gguf_n_kv": (C.c_int, [C.c_void_p]),
    "msq_gguf_alignment": (C.c_uint32, [C.c_void_p]),
    "msq_gguf_version": (C.c_uint32, [C.c_void_p]),
    "msq_gguf_split_path": (C.c_char_p, [C.c_void_p, C.c_int]),
    "msq_gguf_data_offset": (C.c_uint64, [C.c_void_p, C.c_int]),
    "msq_gguf_split_count_of_path": (C.c_int, [C.c_char_p]),
    "msq_gguf_type_bytes": (C.c_uint64, [C.c_int, C.c_uint64]),
    "msq_gguf_type_name": (C.c_char_p, [C.c_int]),
    "msq_gguf_tensor": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(MsqGgufTensor)]),
    "msq_gguf_find": (C.c_int, [C.c_void_p, C.c_char_p]),
    "msq_gguf_key": (C.c_char_p, [C.c_void_p, C.c_int]),
    "msq_gguf_kv_type": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_int)]),
    "msq_gguf_get_i64": (C.c_int64, [C.c_void_p, C.c_char_p, C.c_int64]),
    "msq_gguf_get_f64": (C.c_double, [C.c_void_p, C.c_char_p, C.c_double]),
    "msq_gguf_get_str": (C.c_char_p, [C.c_void_p, C.c_char_p, C.c_char_p]),
    "msq_gguf_arr_len": (C.c_int64, [C.c_void_p, C.c_char_p]),
    "msq_gguf_arr_i64": (C.c_int64, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int64]),
    "msq_gguf_arr_f64": (C.c_int64, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int64]),
    "msq_gguf_arr_str": (C.c_char_p, [C.c_void_p, C.c_char_p, C.c_int64]),
    "msq_gguf_arr_nested_i64": (C.c_int64, [C.c_void_p, C.c_char_p, C.c_int64, C.c_void_p, C.c_int64]),
    "msq_gguf_read": (C.c_int64, [C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_uint64]),
    "msq_gguf_load_tensor": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, _BP]),
    "msq_gguf_expert_layout": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(MsqExpertLayout)]),
    "msq_gguf_place_experts": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, _BP, C.POINTER(MsqExpertSlot), C.c_int]),
    "msq_route_lists": (C.c_int, [C.c_void_p, _BP, _BP, C.c_int, C.c_int, C.POINTER(MsqRouteLists)]),
}


def load():
    """The loaded library. Raises if libmsq.so has not been built (python -m macseek_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO):
            raise RuntimeError("macseek_amd: %s is missing; build it with `python -m macseek_amd.build` "
                               "(there is no CPU fallback)" % SO)
        L = C.CDLL(SO)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the library does not export a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib
