"""Loads cubert_amd/libcuBERT.so and declares the C ABI of include/*.h to ctypes.

The library is the product: if it is missing the import of anything that needs
it fails with a clear error (there is no CPU or PyTorch fallback).
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcuBERT.so")

_lib = None

vp = ctypes.c_void_p
ci = ctypes.c_int
cf = ctypes.c_float
cll = ctypes.c_longlong


class cuBERT_Output(ctypes.Structure):
    """struct cuBERT_Output of include/cuBERT.h (field order is ABI)."""
    _fields_ = [("logits", vp), ("pooled_output", vp), ("sequence_output", vp), ("embedding_output", vp), ("probs", vp)]


# name -> (restype, argtypes); everything include/*.h declares
SIGNATURES = {
    # include/cuBERT.h
    "cuBERT_initialize": (None, []),
    "cuBERT_finalize": (None, []),
    "cuBERT_get_gpu_count": (ci, []),
    "cuBERT_open": (vp, [ctypes.c_char_p, ci, ci, ci, ci, ci]),
    "cuBERT_compute": (None, [vp, ci, vp, vp, vp, vp, ci, ci]),
    "cuBERT_close": (None, [vp, ci]),
    "cuBERT_open_tokenizer": (vp, [ctypes.c_char_p, ci]),
    "cuBERT_close_tokenizer": (None, [vp]),
    "cuBERT_tokenize_compute": (None, [vp, vp, ci, vp, vp, vp, ci, ci]),
    "cuBERT_compute_m": (None, [vp, ci, vp, vp, vp, ctypes.POINTER(cuBERT_Output), ci, ci]),
    "cuBERT_tokenize_compute_m": (None, [vp, vp, ci, vp, vp, ctypes.POINTER(cuBERT_Output), ci, ci]),
    # include/cubert_host.h
    "cubert_last_error": (ctypes.c_char_p, []),
    "cubert_try_open": (ci, [ctypes.c_char_p, ci, ci, ci, ci, ci, ctypes.POINTER(vp)]),
    "cubert_try_compute": (ci, [vp, ci, vp, vp, vp, vp, ci, ci]),
    "cubert_try_compute_m": (ci, [vp, ci, vp, vp, vp, ctypes.POINTER(cuBERT_Output), ci, ci]),
    "cubert_try_close": (ci, [vp, ci]),
    "cubert_model_info": (ci, [vp, ci, ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.POINTER(ci)]),
    "cubert_check_input_range": (ci, [vp, vp, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t]),
    "cubert_open_warmup_batches": (cll, [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t),
                                         ctypes.c_size_t]),
    "cubert_graph_open": (ci, [ctypes.c_char_p, ci, ctypes.POINTER(vp)]),
    "cubert_graph_count": (cll, [vp, ci]),
    "cubert_graph_var": (vp, [vp, ci, ctypes.c_char_p, ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(cll), ci,
                              ctypes.POINTER(ci)]),
    "cubert_graph_sizes": (ci, [vp, ci, ctypes.POINTER(ctypes.c_size_t)]),
    "cubert_graph_close": (ci, [vp, ci]),
    "cubert_try_open_tokenizer": (ci, [ctypes.c_char_p, ci, ctypes.POINTER(vp)]),
    "cubert_try_tokenize_compute": (ci, [vp, vp, ci, vp, vp, vp, ci, ci]),
    "cubert_try_tokenize_compute_m": (ci, [vp, vp, ci, vp, vp, ctypes.POINTER(cuBERT_Output), ci, ci]),
    "cubert_tokenizer_tokenize": (ci, [vp, ci, ctypes.c_char_p, ci, vp, ctypes.c_size_t, ctypes.POINTER(ci),
                                       ctypes.POINTER(ctypes.c_size_t)]),
    "cubert_tokenizer_wordpiece": (ci, [vp, ctypes.c_char_p, vp, ctypes.c_size_t, ctypes.POINTER(ci),
                                        ctypes.POINTER(ctypes.c_size_t)]),
    "cubert_tokenizer_token_id": (ctypes.c_longlong, [vp, ctypes.c_char_p]),
    "cubert_tokenizer_convert_example": (ci, [vp, ci, ctypes.c_char_p, ctypes.c_char_p, vp, vp, vp]),
    "cubert_tokenizer_char_class": (ci, [ci, ci]),
    "cubert_tokenizer_nfd": (ci, [ctypes.c_char_p, vp, ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t)]),
    "cubert_tokenizer_unicode_version": (ctypes.c_char_p, []),
    "cubert_bert_create": (ci, [ci, ci, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(vp), ci, ci, ci, ci, ci, ci, ci,
                                ci, ci, ctypes.POINTER(vp)]),
    "cubert_bert_compute": (ci, [vp, ci, ci, vp, vp, vp]),
    "cubert_bert_output": (ci, [vp, ci, ci, ctypes.POINTER(cuBERT_Output), ci]),
    "cubert_bert_stream": (vp, [vp, ci]),
    "cubert_bert_compute_resident": (ci, [vp, ci, ci]),
    "cubert_bert_profile": (ci, [vp, ci, ctypes.c_uint]),
    "cubert_bert_profile_read": (ci, [vp, ci, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ci), ci]),
    "cubert_bert_destroy": (ci, [vp, ci]),
    "cubert_transformer_run": (ci, [ci, ctypes.c_char_p, ci, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(vp), ci, ci,
                                    ci, ci, ci, ci, vp, vp, vp]),
    # include/cubert_kernels.h: runtime
    "cubert_get_gpu_count": (ci, []),
    "cubert_set_gpu": (ci, [ci]),
    "cubert_gpu_info": (ci, [ci]),
    "cubert_malloc": (vp, [ctypes.c_size_t]),
    "cubert_free": (ci, [vp]),
    "cubert_mem_info": (ci, [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
    "cubert_memcpy": (ci, [vp, vp, ctypes.c_size_t, ci]),
    "cubert_memcpy_async": (ci, [vp, vp, ctypes.c_size_t, ci, vp]),
    "cubert_stream_create": (vp, []),
    "cubert_stream_destroy": (ci, [vp]),
    "cubert_stream_synchronize": (ci, [vp]),
    "cubert_malloc_host": (vp, [ctypes.c_size_t]),
    "cubert_free_host": (ci, [vp]),
    "cubert_event_synchronize": (ci, [vp]),
    "cubert_event_create": (vp, []),
    "cubert_event_destroy": (ci, [vp]),
    "cubert_event_record": (ci, [vp, vp]),
    "cubert_event_elapsed_ms": (ci, [vp, vp, ctypes.POINTER(cf)]),
    "cubert_time_next_launch": (ci, [vp, vp]),
    "cubert_attention_order": (ci, [vp, ci, ci, vp, vp]),
    "cubert_attention_fused_ordered_f32": (ci, [vp, vp, vp, ci, vp, vp, vp, ci, cf, ci, ci, ci, ci, vp]),
    "cubert_attention_fused_ordered_f16": (ci, [vp, vp, vp, ci, vp, vp, vp, ci, cf, ci, ci, ci, ci, vp]),
    "cubert_gemm_skinny_noalloc_f32": (ci, [vp, ci, ci, ci, cf, vp, ci, vp, ci, vp, ci, vp, ci]),
    "cubert_gemm_skinny_packed_elements": (ctypes.c_size_t, [ci, ci]),
    "cubert_gemm_f16_f32": (ci, [vp, ci, ci, ci, ci, ci, cf, vp, ci, vp, ci, cf, vp, ci, vp]),
    "cubert_split3_f32": (ci, [vp, ci, ci, cf, ci, vp, vp, vp]),
    "cubert_bias_gelu_split3_f32": (ci, [vp, vp, ci, ci, cf, vp, vp, vp]),
    "cubert_attention_fused_split3_f32": (ci, [vp, vp, vp, ci, vp, cf, vp, cf, ci, ci, ci, ci, vp, vp]),
    "cubert_bias_res_ln_split3_f32": (ci, [vp, vp, vp, vp, vp, ci, ci, cf, vp, vp, vp]),
    "cubert_blas_create": (vp, []),
    "cubert_blas_destroy": (ci, [vp]),
    "cubert_blas_set_stream": (ci, [vp, vp]),
    "cubert_blas_get_stream": (vp, [vp]),
}
for _t in ("f32", "f16"):
    SIGNATURES.update({
        "cubert_gather_" + _t: (ci, [vp, ci, vp, ci, vp, vp]),
        "cubert_gather_i8_" + _t: (ci, [vp, ci, vp, ci, vp, vp]),
        "cubert_embed_ln_" + _t: (ci, [vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, vp]),
        "cubert_bias_res_ln_" + _t: (ci, [vp, vp, vp, vp, vp, ci, ci, vp]),
        "cubert_bias_gelu_" + _t: (ci, [vp, vp, ci, ci, vp]),
        "cubert_mask_scale_softmax_" + _t: (ci, [vp, vp, cf, ci, ci, ci, vp]),
        "cubert_row_softmax_" + _t: (ci, [vp, vp, ci, ci, vp]),
        "cubert_attention_scores_" + _t: (ci, [vp, vp, ci, vp, cf, ci, ci, ci, ci, vp]),
        "cubert_attention_fused_" + _t: (ci, [vp, vp, vp, ci, vp, vp, ci, cf, ci, ci, ci, ci, vp]),
        "cubert_attention_context_" + _t: (ci, [vp, vp, ci, vp, ci, ci, ci, ci, ci, vp]),
        "cubert_bias_tanh_" + _t: (ci, [vp, vp, ci, ci, vp]),
        "cubert_mean_pool_" + _t: (ci, [vp, vp, ci, ci, ci, vp]),
        "cubert_transpose_" + _t: (ci, [vp, ci, ci, vp, vp]),
        "cubert_classifier_head_" + _t: (ci, [vp, vp, vp, vp, vp, vp, ci, ci, ci, vp]),
        "cubert_gemm_" + _t: (ci, [vp, ci, ci, ci, ci, ci, cf, vp, ci, vp, ci, cf, vp, ci, vp]),
        "cubert_gemm_skinny_" + _t: (ci, [vp, ci, ci, ci, cf, vp, ci, vp, ci, vp, ci, vp, ci]),
        "cubert_gemm_skinny_pack_" + _t: (ci, [vp, vp, ci, ci, ci, vp]),
        "cubert_gemm_skinny_packed_" + _t: (ci, [vp, ci, ci, ci, cf, vp, vp, ci, vp, ci, vp, ci]),
        "cubert_gemm_skinny_partials_" + _t: (ci, [vp, ci, ci, ci, vp, ci, ci, vp, ci, vp, ctypes.c_size_t,
                                                  ctypes.POINTER(ci), ctypes.POINTER(ci)]),
        "cubert_bias_res_ln_partials_" + _t: (ci, [vp, vp, ci, ci, vp, vp, vp, vp, ci, ci, vp]),
        "cubert_gemm_strided_batch_" + _t: (ci, [vp, ci, ci, ci, ci, ci, cf, vp, ci, cll, vp, ci, cll, cf, vp, ci, cll, ci]),
        "cubert_gemm_batch_" + _t: (ci, [vp, ci, ci, ci, ci, ci, cf, vp, ci, vp, ci, cf, vp, ci, ci]),
    })


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m cubert_amd.build` "
                               "(there is no fallback path)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if a declared symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib
