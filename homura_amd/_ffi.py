"""ctypes binding of libhomura_amd.so — the C boundary declared in include/homura_amd.h.

The library is loaded from the package directory and never built implicitly: if it is
missing the import of any GPU entry point fails loudly (run `python -m homura_amd.build`).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libhomura_amd.so"

c_void_pp = C.POINTER(C.c_void_p)
c_f32_p = C.POINTER(C.c_float)


class HmTransformerConfig(C.Structure):
    _fields_ = [
        ("hidden_size", C.c_int),
        ("intermediate_size", C.c_int),
        ("num_attention_heads", C.c_int),
        ("num_hidden_layers", C.c_int),
        ("num_key_value_heads", C.c_int),
        ("vocab_size", C.c_int),
        ("head_dim", C.c_int),
        ("max_position_embeddings", C.c_int),
        ("tie_word_embeddings", C.c_int),
        ("rms_norm_eps", C.c_double),
        ("rope_theta", C.c_double),
        ("attention_bias", C.c_int),
        ("eos_token_id", C.c_int),
        ("bos_token_id", C.c_int),
    ]


class HmSamplingConfig(C.Structure):
    _fields_ = [
        ("temperature", C.c_float),
        ("top_k", C.c_int),
        ("top_p", C.c_float),
        ("min_p", C.c_float),
        ("repetition_penalty", C.c_float),
        ("frequency_penalty", C.c_float),
        ("presence_penalty", C.c_float),
    ]


class HmKernelProfile(C.Structure):
    _fields_ = [
        ("label", C.c_char * 32),
        ("ms", C.c_float),
        ("launches", C.c_int),
        ("bytes", C.c_double),
    ]


_P = C.c_void_p
_I = C.c_int
_SZ = C.c_size_t

# name -> (restype, argtypes); mirrors include/homura_amd.h one to one
SIGNATURES = {
    "hm_init": (_P, [_I]),
    "hm_destroy": (None, [_P]),
    "hm_last_error": (C.c_char_p, [_P]),
    "hm_alloc": (_I, [_P, _SZ, c_void_pp]),
    "hm_free": (_I, [_P, _P]),
    "hm_upload": (_I, [_P, _P, _P, _SZ]),
    "hm_download": (_I, [_P, _P, _P, _SZ]),
    "hm_copy": (_I, [_P, _P, _P, _SZ]),
    "hm_fill_zero": (_I, [_P, _P, _SZ]),
    "hm_sync": (_I, [_P]),
    "hm_stream": (_P, [_P]),
    "hm_device_name": (_I, [_P, C.c_char_p, _SZ]),
    "hm_event_create": (_I, [_P, c_void_pp]),
    "hm_event_destroy": (_I, [_P, _P]),
    "hm_event_record": (_I, [_P, _P]),
    "hm_event_elapsed_ms": (_I, [_P, _P, _P, c_f32_p]),
    "hm_graph_begin": (_I, [_P]),
    "hm_graph_end": (_I, [_P, c_void_pp]),
    "hm_graph_launch": (_I, [_P, _P, _I]),
    "hm_graph_destroy": (_I, [_P, _P]),
    "hm_gemv_bf16": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_pack_bf16_kn_to_nk": (_I, [_P, _P, _P, _I, _I]),
    "hm_gemv_bf16_nk": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemv_q8_0": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemv_q4_0": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_quant_planes_bytes": (_SZ, [_I, _I, _I]),
    "hm_pack_quant_planes": (_I, [_P, _I, _P, _P, _I, _I]),
    "hm_unpack_quant_planes": (_I, [_P, _I, _P, _P, _I, _I]),
    "hm_gemv_q8_0_planes": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemv_q4_0_planes": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_dequant_quant_planes": (_I, [_P, _I, _P, _P, _I, _I]),
    "hm_gemv_q6_k_f32_planes": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_test_fill_lds": (_I, [_P, C.c_uint32]),
    "hm_dequant_q8_0": (_I, [_P, _P, _P, _SZ]),
    "hm_dequant_q4_0": (_I, [_P, _P, _P, _SZ]),
    "hm_gemv_q4_k": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemv_q6_k": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_k8_bytes": (_SZ, [_I, _I]),
    "hm_pack_k8": (_I, [_P, _I, _P, _I, _P, _I, _I, _I]),
    "hm_gemv_k8": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemv_q4_k_f32": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemv_q6_k_f32": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_quantize_q8_k": (_I, [_P, _P, _P, _P, _P, _I, _I]),
    "hm_dequant_q4_k": (_I, [_P, _P, _P, _SZ]),
    "hm_dequant_q6_k": (_I, [_P, _P, _P, _SZ]),
    "hm_gemm_bf16": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemm_bf16_nk": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemm_f32_bf16_nk": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_gemm_f32_quant_nk": (_I, [_P, _P, _P, _I, _P, _I, _I, _I]),
    "hm_model_set_weight_nk": (_I, [_P, _I, _P, _SZ]),
    "hm_model_set_lm_head_blocks": (_I, [_P, _I, _P, _SZ]),
    "hm_model_config": (_I, [_P, _P, _P, _P]),
    "hm_tokenizer_open": (_P, [C.c_char_p, C.c_char_p, C.c_char_p, _SZ]),
    "hm_tokenizer_open_json": (_P, [C.c_char_p, C.c_char_p, _SZ]),
    "hm_tokenizer_close": (None, [_P]),
    "hm_tokenizer_wants_nfc": (_I, [_P]),
    "hm_tokenizer_token_to_id": (C.c_longlong, [_P, C.c_char_p]),
    "hm_tokenizer_encode_ex": (C.c_longlong, [_P, C.c_char_p, _SZ, _I, _P, _SZ]),
    "hm_tokenizer_decode_ex": (C.c_longlong, [_P, _P, _SZ, _I, _P, _SZ]),
    "hm_tokenizer_vocab_size": (_I, [_P]),
    "hm_tokenizer_encode": (C.c_longlong, [_P, C.c_char_p, _SZ, _P, _SZ]),
    "hm_tokenizer_decode": (C.c_longlong, [_P, _P, _SZ, _P, _SZ]),
    "hm_tokenizer_pieces": (C.c_longlong, [C.c_char_p, _SZ, _P, _SZ]),
    "hm_gguf_open": (_P, [C.c_char_p, C.c_char_p, _SZ]),
    "hm_gguf_close": (None, [_P]),
    "hm_gguf_version": (_I, [_P]),
    "hm_gguf_num_tensors": (_I, [_P]),
    "hm_gguf_data_offset": (_SZ, [_P]),
    "hm_gguf_tensor_info": (_I, [_P, _I, C.c_char_p, _SZ, _P, _P, _P, _P, _P]),
    "hm_gguf_find_tensor": (_I, [_P, C.c_char_p]),
    "hm_gguf_tensor_data": (_P, [_P, _I]),
    "hm_gguf_tensor_f32": (_I, [_P, _I, _P, _SZ, C.c_char_p, _SZ]),
    "hm_gguf_meta_str": (_I, [_P, C.c_char_p, C.c_char_p, _SZ]),
    "hm_gguf_meta_u64": (_I, [_P, C.c_char_p, _P]),
    "hm_gguf_meta_f32": (_I, [_P, C.c_char_p, _P]),
    "hm_gguf_meta_array_len": (C.c_int64, [_P, C.c_char_p]),
    "hm_gguf_transformer_config": (_I, [_P, _P, _P, C.c_char_p, _SZ]),
    "hm_safetensors_open": (_P, [C.c_char_p, C.c_char_p, _SZ]),
    "hm_safetensors_close": (None, [_P]),
    "hm_safetensors_num_tensors": (_I, [_P]),
    "hm_safetensors_tensor_info": (_I, [_P, _I, C.c_char_p, _SZ, C.c_char_p, _P, _P, _P]),
    "hm_safetensors_tensor_data": (_P, [_P, _I]),
    "hm_config_from_json": (_I, [C.c_char_p, _P, C.c_char_p, _SZ]),
    "hm_model_load_gguf": (_P, [_P, C.c_char_p, _I]),
    "hm_model_load_hf_dir": (_P, [_P, C.c_char_p, _I]),
    "hm_ciface_bind_transformer": (_I, [_P, _P, _I]),
    "hm_ciface_bind_transformer_quant": (_I, [_P, _P, _P, _I]),
    "hm_ciface_num_kernels": (_I, []),
    "hm_ciface_unbind": (None, []),
    "hm_ciface_last_status": (_I, [C.POINTER(C.c_int)]),
    "hm_ciface_clear_status": (None, []),
    "hm_kv_append": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I]),
    "hm_gqa_decode_attn": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, C.c_float]),
    "hm_gqa_decode_attn_noalloc": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, C.c_float]),
    "hm_gqa_decode_attn_noalloc_limit": (_SZ, []),
    "hm_gqa_prefill_attn": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, C.c_float]),
    "hm_rmsnorm": (_I, [_P, _P, _P, _P, _I, _I, C.c_float]),
    "hm_qknorm_rope": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, C.c_float]),
    "hm_silu_mul": (_I, [_P, _P, _P, _P, _SZ]),
    "hm_add": (_I, [_P, _P, _P, _P, _SZ]),
    "hm_embed": (_I, [_P, _P, _P, _P, _I, _I, _I]),
    "hm_argmax": (_I, [_P, _P, _I, _P]),
    "hm_model_create": (_P, [_P, C.POINTER(HmTransformerConfig), _I, _I]),
    "hm_model_create_mixed": (_P, [_P, C.POINTER(HmTransformerConfig), C.POINTER(_I), _I]),
    "hm_model_destroy": (None, [_P]),
    "hm_model_num_weight_slots": (_I, [_P]),
    "hm_model_weight_slot_info": (_I, [_P, _I, C.c_char_p, _SZ, C.POINTER(_I),
                                       C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                       C.POINTER(_SZ)]),
    "hm_model_set_weight": (_I, [_P, _I, _P, _SZ]),
    "hm_model_finalize": (_I, [_P, _I]),
    "hm_model_init_kv_cache": (_I, [_P, C.POINTER(c_f32_p), _I]),
    "hm_model_reset_kv_cache": (_I, [_P]),
    "hm_model_kv_cache_len": (_I, [_P]),
    "hm_model_set_graph": (_I, [_P, _I]),
    "hm_model_set_whole_step": (_I, [_P, _I]),
    "hm_model_whole_step": (_I, [_P]),
    "hm_model_whole_step_available": (_I, [_P]),
    "hm_model_whole_step_status": (_I, [_P]),
    "hm_model_whole_step_inject_timeout": (_I, [_P, _I, _I]),
    "hm_model_whole_step_trace": (_I, [_P, _P, _I, C.POINTER(C.c_int)]),
    "hm_model_prefill_capture_q8k_inputs": (_I, [_P, _I]),
    "hm_model_prefill_captured_q8k_inputs": (_I, [_P, _P, _SZ]),
    "hm_model_run_kv": (_I, [_P, C.POINTER(C.c_int64), _I, c_f32_p]),
    "hm_model_prefill": (_I, [_P, C.POINTER(C.c_int64), _I, c_f32_p]),
    "hm_model_generate": (_I, [_P, C.POINTER(C.c_int64), _I, _I, C.POINTER(HmSamplingConfig), C.c_uint64, _I,
                               C.POINTER(C.c_int32), C.POINTER(_I)]),
    "hm_rng_seed": (C.c_uint64, [C.c_uint64]),
    "hm_rng_next_f32": (C.c_float, [C.POINTER(C.c_uint64)]),
    "hm_sample_token_host": (_I, [_P, _I, C.POINTER(HmSamplingConfig), _P, _I, C.POINTER(C.c_uint64),
                                  C.POINTER(C.c_int32)]),
    "hm_sample_token": (_I, [_P, _P, _I, C.POINTER(HmSamplingConfig), _P, _I, C.POINTER(C.c_uint64),
                             C.POINTER(C.c_int32)]),
    "hm_model_set_prefill_min": (_I, [_P, _I]),
    "hm_model_set_prefill_pieces": (_I, [_P, _I]),
    "hm_model_set_prefill_weight_cache": (_I, [_P, _SZ]),
    "hm_model_generate_greedy": (_I, [_P, C.POINTER(C.c_int64), _I, _I, C.POINTER(C.c_int32)]),
    "hm_model_bench_decode": (_I, [_P, C.c_int64, _I, c_f32_p, C.POINTER(C.c_int32)]),
    "hm_model_profile_step": (_I, [_P, C.c_int64, C.POINTER(HmKernelProfile), _I]),
    "hm_model_time_kernels": (_I, [_P, _I, C.POINTER(HmKernelProfile), _I]),
    "hm_model_launches_per_step": (_I, [_P]),
    "hm_bench_launch_floor": (_I, [_P, _I, _I, _I, c_f32_p]),
    "hm_synth_normal_f32": (None, [C.c_uint64, C.c_uint64, _SZ, C.c_float, _P]),
    "hm_synth_normal_bf16": (None, [C.c_uint64, C.c_uint64, _SZ, C.c_float, _P]),
    "hm_synth_token_ids": (None, [C.c_uint64, _SZ, _I, _P]),
    "hm_synth_q8_0": (None, [C.c_uint64, _SZ, C.c_float, _P]),
    "hm_synth_q4_0": (None, [C.c_uint64, _SZ, C.c_float, _P]),
    "hm_f32_to_bf16_rne": (C.c_uint16, [C.c_float]),
    "hm_f32_to_f16_rne": (C.c_uint16, [C.c_float]),
    "hm_version": (C.c_char_p, []),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library and attach the signatures. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it first with `python -m homura_amd.build` "
            "(there is no CPU fallback)")
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library out of step
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
