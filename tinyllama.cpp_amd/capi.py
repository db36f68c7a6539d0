"""ctypes binding of the C-ABI in include/tlhip.h (csrc/libtlhip.so).

There is NO fallback: if the library is missing or a call fails, an exception is raised (TlError carries
tl_last_error()). Nothing here touches the CPU oracle.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "csrc", "libtlhip.so")

F32, Q8_0, Q4_K, Q6_K, Q8_K = 0, 8, 12, 14, 15
(T_ATTN_Q, T_ATTN_K, T_ATTN_V, T_ATTN_OUTPUT, T_FFN_GATE, T_FFN_UP, T_FFN_DOWN, T_ATTN_NORM, T_FFN_NORM,
 T_TOKEN_EMBD, T_OUTPUT_NORM, T_OUTPUT) = range(12)


class TlError(RuntimeError):
    pass


class ModelConfig(C.Structure):
    _fields_ = [("hidden_size", C.c_int), ("intermediate_size", C.c_int), ("num_attention_heads", C.c_int),
                ("num_key_value_heads", C.c_int), ("num_hidden_layers", C.c_int), ("vocab_size", C.c_int),
                ("max_position_embeddings", C.c_int), ("rms_norm_eps", C.c_float), ("rope_theta", C.c_float),
                ("tp_rank", C.c_int), ("tp_size", C.c_int)]


class LayerSpec(C.Structure):
    pass


LayerSpec._fields_ = [("mixer", C.c_int), ("heads", C.c_int), ("kv_heads", C.c_int), ("dim", C.c_int), ("vdim", C.c_int),
                ("window", C.c_int), ("scale", C.c_float), ("qk_norm", C.c_int), ("v_mix", C.c_int), ("mlp", C.c_int),
                ("experts", C.c_int), ("top", C.c_int), ("expert_ff", C.c_int), ("expert_limit", C.c_float),
                ("shared_ff", C.c_int), ("shared_limit", C.c_float), ("act_alpha", C.c_float),
                ("glu_up_add", C.c_float), ("block", C.c_int), ("weights_of", C.c_int), ("keep_first", C.c_int),
                ("attn_weight", C.c_int), ("values_are_keys", C.c_int), ("rot_dims", C.c_int), ("rot_base", C.c_float),
                ("rot_factor", C.c_float), ("rot_original", C.c_float), ("rot_fast", C.c_float), ("rot_slow", C.c_float),
                ("conv_taps", C.c_int), ("decay_rank", C.c_int), ("gate_rank", C.c_int), ("route", C.c_int),
                ("route_groups", C.c_int), ("route_keep", C.c_int), ("shared_gate", C.c_int), ("q_temp_coef", C.c_float),
                ("q_temp_every", C.c_int), ("q_rank", C.c_int), ("kv_rank", C.c_int), ("rot_dim", C.c_int),
                ("kv_from", C.c_int), ("head_gate", C.c_int), ("decay_scale", C.c_float), ("act", C.c_int),
                ("glu", C.c_int), ("score_maps", C.c_int), ("diff_init", C.c_float), ("out_gate", C.c_int),
                ("qkv_bias", C.c_int), ("qkv_conv", C.c_int), ("score_softcap", C.c_float), ("dist_bias", C.c_int),
                ("decay_per_head", C.c_int), ("side", C.POINTER(LayerSpec)), ("mix_scale", C.c_float),
                ("side_scale", C.c_float)]


class StackConfig(C.Structure):
    _fields_ = [("width", C.c_int), ("vocab", C.c_int), ("n_layers", C.c_int), ("max_positions", C.c_int),
                ("norm_eps", C.c_float), ("layers", C.POINTER(LayerSpec)), ("norm", C.c_int), ("embed_norm", C.c_int),
                ("logit_softcap", C.c_float), ("embed_scale", C.c_float), ("canon_taps", C.c_int)]


BF16 = 30
LAYER_HOOK = C.CFUNCTYPE(None, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int)

_vp, _fp, _ip, _sz = C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t  # device pointers travel as integers

# name -> argtypes; every symbol include/tlhip.h declares (tests/test_capi_symbols.py checks the two agree)
SIGNATURES = {
    "tl_init": [C.c_int],
    "tl_device_count": [C.POINTER(C.c_int)],
    "tl_malloc": [C.POINTER(C.c_void_p), _sz],
    "tl_shutdown": [],
    "tl_free": [_vp],
    "tl_memset": [_vp, C.c_int, _sz, _vp],
    "tl_memcpy_h2d": [_vp, _vp, _sz, _vp],
    "tl_memcpy_d2h": [_vp, _vp, _sz, _vp],
    "tl_memcpy_d2d": [_vp, _vp, _sz, _vp],
    "tl_stream_create": [C.POINTER(C.c_void_p)],
    "tl_stream_destroy": [_vp],
    "tl_stream_sync": [_vp],
    "tl_device_sync": [],
    "tl_qweight_upload": [C.c_int, _vp, C.c_int, C.c_int, C.POINTER(C.c_void_p), _vp],
    "tl_qweight_free": [_vp],
    "tl_qweight_info": [_vp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(_sz)],
    "tl_qweight_expand": [_vp, C.POINTER(_sz), _vp],
    "tl_dequantize_rows": [_vp, C.c_int, C.c_int, _fp, _vp],
    "tl_matvec_q": [_vp, _fp, _fp, _vp],
    "tl_matmul_q": [_vp, _fp, _fp, C.c_int, _vp],
    "tl_rmsnorm_vector": [_fp, _fp, _fp, C.c_int, C.c_float, _vp],
    "tl_rmsnorm_batch": [_fp, _fp, _fp, C.c_int, C.c_int, C.c_float, _vp],
    "tl_rope_table_upload": [_fp, C.c_int, C.c_int, C.c_float, _vp],
    "tl_rope": [_fp, C.c_int, C.c_int, _fp, C.c_int, C.c_int, C.c_int, _vp],
    "tl_rope_batch": [_fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp],
    "tl_update_kv_cache": [_fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp],
    "tl_update_kv_cache_batch": [_fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp],
    "tl_attention": [_fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int, _vp],
    "tl_attention_noalloc": [_fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int, _vp],
    "tl_attention_batch_prefill": [_fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                   C.c_float, _vp],
    "tl_add_residual": [_fp, _fp, _fp, _sz, _vp],
    "tl_swiglu": [_fp, _fp, _fp, _sz, C.c_int, _vp],
    "tl_lookup_embedding": [_vp, C.c_int, _fp, _vp],
    "tl_argmax": [_fp, C.c_int, _ip, _vp],
    "tl_model_create": [C.POINTER(ModelConfig), C.POINTER(C.c_void_p)],
    "tl_model_free": [_vp],
    "tl_model_set_tensor": [_vp, C.c_int, C.c_int, C.c_int, _vp, C.c_int, C.c_int],
    "tl_model_finalize": [_vp],
    "tl_model_reset_kv": [_vp],
    "tl_model_decode": [_vp, C.c_int, C.c_int, _vp, C.POINTER(C.c_int)],
    "tl_model_generate_greedy": [_vp, C.c_int, C.c_int, C.c_int, C.c_float, _vp, C.c_int, _vp],
    "tl_model_prefill": [_vp, _vp, C.c_int, C.c_int, _vp, _vp],
    "tl_quantize_q8_k": [_vp, _sz, _vp, _vp],
    "tl_model_set_prefill": [_vp, C.c_int, C.c_int],
    "tl_model_generate_sampled": [_vp, C.c_int, C.c_int, C.c_int, C.c_float, _vp, C.c_int, C.c_float, C.c_int, C.c_float,
                                  C.c_uint64, _vp],
    "tl_sample_top_k_top_p": [_vp, C.c_int, C.c_float, C.c_int, C.c_float, C.c_float, _vp, _vp, _vp, _vp, _vp],
    "tl_gemm_set_terms": [C.c_int],
    "tl_model_device_ptr": [_vp, C.c_int, C.c_int, C.POINTER(C.c_void_p)],
    "tl_model_bytes_per_token": [_vp, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "tl_model_prefill_planes_bytes": [_vp, C.POINTER(_sz)],
    "tl_tp_unique_id": [_vp],
    "tl_tp_local_group_prefill": [_vp, C.c_int, _vp, C.c_int, C.c_int, _vp],
    "tl_model_graph_captured": [_vp, _vp],
    "tl_model_batch_init": [_vp, C.c_int],
    "tl_model_batch_prefill": [_vp, C.c_int, _vp, C.c_int, C.c_int, _vp],
    "tl_model_batch_decode": [_vp, C.c_int, _vp, _vp, _vp, _vp, _vp],
    "tl_model_batch_prefill_packed": [_vp, C.c_int, _vp, _vp, _vp, C.c_int, _vp, _vp, _vp],
    "tl_model_batch_generate_greedy": [_vp, C.c_int, _vp, _vp, _vp, C.c_int, _vp],
    "tl_model_tp_init": [_vp, _vp],
    "tl_model_tp_peer_export": [_vp, _vp],
    "tl_model_tp_peer_import": [_vp, _vp, _vp],
    "tl_model_tp_peer_enable": [_vp, C.c_int],
    "tl_model_tp_peer_enabled": [_vp, _vp],
    "tl_model_tp_peer_fused": [_vp, _vp],
    "tl_model_graph_nodes": [_vp, _vp],
    "tl_tp_local_group_decode": [_vp, C.c_int, C.c_int, C.c_int, _vp, C.POINTER(C.c_int)],
    "tl_model_create_stack": [C.POINTER(StackConfig), C.POINTER(C.c_void_p)],
    "tl_model_set_tensor_named": [_vp, C.c_char_p, C.c_int, C.POINTER(C.c_longlong), C.c_int, _vp],
    "tl_model_prefill_rows": [_vp, _vp, C.c_int, C.c_int, _vp, C.c_int, _vp],
    "tl_dense_matmul": [_vp, C.c_int, C.c_int, _fp, _fp, C.c_int, C.c_int, _vp],
    "tl_swa_attention": [_fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, _vp],
    "tl_resid_rmsnorm": [_fp, _fp, _fp, C.c_int, C.c_int, C.c_float, _vp],
    "tl_moe_route": [_fp, C.c_int, C.c_int, _vp, _fp, C.c_int, C.c_int, _ip, _fp, _vp],
    "tl_glu_clamp": [_fp, C.c_int, C.c_int, C.c_float, C.c_float, _fp, _vp],
    "tl_window_attention": [_fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                            C.c_float, C.c_int, _fp, _vp],
    "tl_moe_route_groups": [_fp, C.c_int, C.c_int, _vp, C.c_int, C.c_int, C.c_int, C.c_int, _ip, _fp, _vp],
    "tl_dyt_norm": [_fp, _fp, _fp, _fp, _fp, C.c_int, C.c_int, _vp],
    "tl_rotary_heads": [_fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_float,
                        C.c_float, C.c_int, C.c_float, _vp],
    "tl_delta_prepare": [_fp, C.c_int, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp, _fp, _fp, _fp, _fp,
                         _fp, _fp, _vp],
    "tl_delta_rule": [_fp, _fp, _fp, _fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp],
    "tl_gated_head_norm": [_fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_float, _vp],
    "tl_window_attention_rows": [_fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                 C.c_int, C.c_int, C.c_float, C.c_int, _fp, _vp],
    "tl_layer_norm": [_fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_float, _vp],
    "tl_dense_matmul_act": [_vp, C.c_int, C.c_int, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_int, _vp],
    "tl_dense_matmul_heads": [_vp, C.c_int, C.c_int, C.c_int, _fp, C.c_int, C.c_int, _fp, C.c_int, C.c_int, C.c_int, C.c_int,
                              _vp],
    "tl_causal_conv": [_fp, C.c_int, C.c_int, C.c_int, C.c_int, _fp, _vp, _fp, C.c_int, C.c_int, _fp, C.c_int, _vp],
    "tl_moe_route_sigmoid_groups": [_fp, C.c_int, C.c_int, _vp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, _ip, _fp, _vp],
    "tl_window_attention_opts": [_fp, C.c_int, C.c_int, _fp, C.c_int, C.c_int, _fp, C.c_int, _fp, C.c_int, C.c_int, C.c_int,
                                 C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, _fp, _fp, C.c_int, _fp, _vp],
    "tl_head_norm": [_fp, _fp, C.c_float, _fp, C.c_int, C.c_int, _fp, C.c_int, C.c_float, C.c_int, C.c_int, C.c_int,
                     C.c_float, _vp],
    "tl_gated_linear_attention": [_fp, C.c_int, _fp, _fp, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, _vp],
    "tl_general_delta": [_fp, C.c_int, _fp, _fp, _fp, C.c_float, _fp, _fp, _fp, C.c_int, C.c_int, C.c_int, _vp],
}

# include/tlhip_debug.h: measurement / diagnostic hooks (not part of the boundary)
DEBUG_SIGNATURES = {
    "tl_bench_matvec": [_vp, C.c_int, _fp, _fp, C.c_int, C.c_int, C.POINTER(C.c_float), _vp],
    "tl_bench_matvec_prefetch": [_vp, C.c_int, _fp, _fp, C.c_int, C.c_int, C.POINTER(C.c_float)],
    "tl_debug_gemv_stamps": [_vp, _fp, _fp, _vp, C.POINTER(C.c_int), C.POINTER(C.c_int), _vp],
    "tl_model_profile_decode": [_vp, C.c_int, C.c_int, C.c_int, _vp, _vp],
    "tl_model_bench_kernel": [_vp, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_double)],
    "tl_chain_set_stamps": [_vp, _sz],
    "tl_debug_gemm_px_launches": [C.POINTER(C.c_longlong)],
    "tl_model_debug_layer_hook": [_vp, LAYER_HOOK, _vp],
}

# libtlhip_tools.so (csrc/tl_stream.hip): experiments kept out of the product library; declared in include/tlhip_debug.h
TOOLS_LIB_PATH = os.path.join(HERE, "csrc", "libtlhip_tools.so")
TOOLS_SIGNATURES = {
    "tl_stream_matvec": [_vp, C.c_int, _fp, _fp, C.c_int, C.POINTER(C.c_float), _vp],
}

_lib = None
_tools_lib = None


def lib():
    """The loaded library with typed entry points; raises if csrc/libtlhip.so has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TlError(f"{LIB_PATH} is missing: build it with `make -C tinyllama.cpp_amd/csrc` "
                          "(or __graft_entry__.build()); there is no CPU fallback")
        L = C.CDLL(LIB_PATH)
        L.tl_last_error.restype = C.c_char_p
        L.tl_last_error.argtypes = []
        for name, argtypes in list(SIGNATURES.items()) + list(DEBUG_SIGNATURES.items()):
            fn = getattr(L, name)
            fn.restype = C.c_int
            fn.argtypes = argtypes
        _lib = L
    return _lib


def tools_lib():
    """libtlhip_tools.so with typed entry points (it links against libtlhip.so, which is loaded first)."""
    global _tools_lib
    if _tools_lib is None:
        lib()
        if not os.path.exists(TOOLS_LIB_PATH):
            raise TlError(f"{TOOLS_LIB_PATH} is missing: build it with `make -C tinyllama.cpp_amd/csrc`")
        L = C.CDLL(TOOLS_LIB_PATH)
        for name, argtypes in TOOLS_SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = C.c_int
            fn.argtypes = argtypes
        _tools_lib = L
    return _tools_lib


def check(rc, what=""):
    if rc != 0:
        raise TlError(f"{what} failed (rc={rc}): {lib().tl_last_error().decode(errors='replace')}")
