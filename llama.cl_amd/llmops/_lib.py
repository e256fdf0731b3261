"""ctypes binding of libllmops_hip.so (the C ABI declared in include/llmops_hip.h)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libllmops_hip.so")

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_f32 = ctypes.c_float
c_ptr = ctypes.c_void_p
c_size = ctypes.c_size_t

# name -> (restype, argtypes); kept in the order of include/llmops_hip.h, then include/llmops_hip_test.h
SIGNATURES = {
    "llmops_last_error": (ctypes.c_char_p, []),
    "llmops_abi_version": (c_int, []),
    "llmops_q4a_block_bytes": (c_i64, [c_int]),
    "llmops_offline_FC_quant_Q4A": (c_int, [c_ptr, c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr]),
    "llmops_offline_FC_dequant_Q4A": (c_int, [c_ptr, c_i64, c_i64, c_int, c_ptr, c_ptr]),
    "llmops_FC_dynamic_quantize_x": (c_int, [c_ptr, c_i64, c_i64, c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "llmops_FC_dynamic_quantize_x_rows": (c_int, [c_ptr, c_i64, c_i64, c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "llmops_fc_Q4A_workspace_bytes": (c_size, [c_i64, c_i64, c_i64, c_i64, c_int]),
    "llmops_fc_Q4A": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_int, c_i64, c_ptr, c_ptr, c_size, c_ptr]),
    "llmops_fc_workspace_reset": (c_int, [c_ptr, c_size, c_ptr]),
    "llmops_fc_Q4A_noalloc_scratch_bytes": (c_size, []),
    "llmops_fc_Q4A_noalloc": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_int, c_i64, c_ptr, c_ptr]),
    "llmops_fc_Q4A_residual": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_int, c_i64, c_ptr, c_ptr, c_ptr, c_size,
                                       c_ptr]),
    "llmops_fc_Q4A_decode": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_int, c_i64, c_ptr, c_f32, c_ptr, c_int, c_ptr,
                                     c_i64, c_ptr, c_ptr, c_ptr, c_size, c_ptr]),
    "llmops_fc_Q4A_decode_parts": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_int, c_i64, c_ptr, c_f32, c_int, c_i64,
                                           c_ptr, c_ptr, c_size, c_ptr]),
    "llmops_fc_Q4A_decode_attn": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_i64, c_ptr, c_ptr, c_ptr, c_ptr,
                                          c_size, c_ptr]),
    "llmops_fc_Q4A_prequantized": (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_ptr, c_i64, c_i64, c_int, c_i64, c_ptr, c_ptr,
                                           c_size, c_ptr]),
    "llmops_fc_Q4A_partials": (c_int, [c_ptr, c_i64, c_ptr, c_i64, c_i64, c_int, c_ptr, c_int, c_ptr]),
    "llmops_rope_embed": (c_int, [c_ptr, c_i64, c_i64, c_i64, c_i64, c_ptr, c_i64, c_int, c_ptr]),
    "llmops_attention_workspace_bytes": (c_size, [c_i64, c_i64, c_i64, c_i64, c_i64]),
    "llmops_attention_rope": (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_ptr, c_i64, c_ptr, c_int,
                                      c_i64, c_i64, c_ptr, c_int, c_int, c_ptr, c_size, c_ptr]),
    "llmops_attention_rope_decode": (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_ptr, c_i64, c_ptr, c_int, c_i64, c_i64,
                                             c_ptr, c_ptr, c_int, c_ptr, c_size, c_ptr]),
    "llmops_attention_records_chunks": (c_i64, [c_i64, c_int]),
    "llmops_attention_records_chunk_rows": (c_i64, [c_i64, c_int]),
    "llmops_attention_rope_decode_records": (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_ptr, c_i64, c_ptr, c_int, c_i64,
                                                     c_i64, c_ptr, c_int, c_ptr, c_int, c_ptr, c_ptr, c_ptr, c_size, c_ptr]),
    "llmops_softmax": (c_int, [c_ptr, c_i64, c_i64, c_ptr]),
    "llmops_mm_qk": (c_int, [c_ptr, c_i64, c_i64, c_i64, c_ptr, c_i64, c_ptr, c_i64, c_i64, c_i64, c_i64, c_i64, c_ptr]),
    "llmops_rmsnorm": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_f32, c_ptr]),
    "llmops_rmsnorm_out": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_ptr, c_f32, c_ptr]),
    "llmops_silu_mul": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_ptr]),
    "llmops_silu_mul_interleaved": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_ptr]),
    "llmops_strip_sumsq": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_ptr]),
    "llmops_iadd": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_int, c_ptr]),
    "llmops_imul": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_int, c_ptr]),
    "llmops_itrans_silu": (c_int, [c_ptr, c_i64, c_ptr]),
    "llmops_embedding_q8c_quant_w": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_ptr, c_ptr]),
    "llmops_embedding_q8c": (c_int, [c_ptr, c_ptr, c_i64, c_ptr, c_ptr, c_i64, c_i64, c_ptr]),
    "llmops_embedding": (c_int, [c_ptr, c_ptr, c_i64, c_ptr, c_i64, c_i64, c_ptr]),
    "llmops_test_calib_read": (c_int, [c_ptr, c_i64, c_int, c_ptr, c_ptr]),
    "llmops_test_calib_copy": (c_int, [c_ptr, c_ptr, c_i64, c_int, c_ptr]),
    "llmops_test_fc_set_tuning": (None, [c_int, c_int]),
    "llmops_test_gemm_set_tuning": (None, [c_int]),
    "llmops_test_gemm_set_reduce": (None, [c_int]),
    "llmops_test_gemm_set_split": (None, [c_int]),
    "llmops_test_gemm_plan": (c_int, [c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr]),
    "llmops_test_fc_set_row_routing": (None, [c_int, c_int]),
    "llmops_test_fc_rows_set_split": (None, [c_int]),
    "llmops_test_attn_set_decode_plan": (None, [c_int]),
    "llmops_test_fc_decode_attn_dump": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_i64, c_ptr, c_ptr, c_ptr, c_ptr,
                                                c_ptr, c_ptr, c_size, c_ptr]),
    "llmops_test_fc_decode_dump": (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_i64, c_i64, c_int, c_i64, c_ptr, c_ptr, c_ptr, c_ptr,
                                           c_ptr, c_ptr, c_size, c_ptr]),
}

_lib = None


def load():
    """Load the shared library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python llama.cl_amd/build.py` (hipcc, gfx950). "
                "llmops has no CPU or eager fallback."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise RuntimeError(load().llmops_last_error().decode())
