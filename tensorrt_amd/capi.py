"""ctypes bindings of the C-ABI kernel layer (include/trtamd_bert_kernels.h).

Functions take raw device addresses (ints) — e.g. ``torch.Tensor.data_ptr()`` — and a stream
handle; nothing here touches torch.  ``check`` turns a non-zero status into an exception carrying
``trtamd_last_error()``.
"""
from __future__ import annotations

import ctypes as C

from . import load_library

c_p = C.c_void_p
i32 = C.c_int32
i64 = C.c_int64
u32 = C.c_uint32
f32 = C.c_float


class FmhaParams(C.Structure):
    """struct trtamd_fmha_params."""
    _fields_ = [
        ("qkv_ptr", c_p), ("packed_mask_ptr", c_p), ("o_ptr", c_p),
        ("qkv_stride_in_bytes", i64), ("packed_mask_stride_in_bytes", i64), ("o_stride_in_bytes", i64),
        ("b", i32), ("h", i32), ("s", i32), ("d", i32),
        ("scale_bmm1", u32), ("scale_softmax", u32), ("scale_bmm2", u32),
        ("enable_i2f_trick", i32),
        ("cu_seqlens", c_p),
        ("interleaved", i32), ("use_int8_scale_max", i32),
        ("warps_m", i32), ("warps_n", i32),
    ]


class Int8LinearParams(C.Structure):
    """struct trtamd_int8_linear_params (include/trtamd_encoder_ops.h)."""
    _fields_ = [
        ("a", c_p), ("w", c_p), ("alpha", c_p), ("beta", c_p), ("out", c_p),
        ("T", i32), ("K", i32), ("N", i32),
        ("a_interleaved", i32), ("w_interleaved", i32), ("out_interleaved", i32), ("epilogue", i32),
        ("out_scale", f32),
    ]


class Fp16LinearParams(C.Structure):
    """struct trtamd_fp16_linear_params (include/trtamd_encoder_ops.h)."""
    _fields_ = [
        ("a", c_p), ("w", c_p), ("alpha", c_p), ("beta", c_p), ("out", c_p),
        ("T", i32), ("K", i32), ("N", i32), ("epilogue", i32),
    ]


LINEAR_AFFINE, LINEAR_GELU, LINEAR_RAW_INT32, LINEAR_AFFINE_FP16 = 0, 1, 2, 3
UNFUSED_ROUTE_ONE_LAUNCH, UNFUSED_ROUTE_THREE_LAUNCHES, UNFUSED_ROUTE_BY_SHAPE = 0, 1, 99


class EncoderConfig(C.Structure):
    """struct trtamd_encoder_config (include/trtamd_encoder_runtime.h)."""
    _fields_ = [("hidden", i32), ("heads", i32), ("ffn", i32), ("layers", i32), ("vocab", i32), ("max_pos", i32),
                ("type_vocab", i32), ("max_seqlen", i32)]


class EncoderEmbedding(C.Structure):
    _fields_ = [("beta", c_p), ("gamma", c_p), ("word", c_p), ("tok", c_p), ("pos", c_p), ("scale", f32)]


class EncoderLinear(C.Structure):
    _fields_ = [("w", c_p), ("alpha", c_p), ("beta", c_p)]


class EncoderLayer(C.Structure):
    _fields_ = [("qkv", EncoderLinear), ("proj", EncoderLinear), ("ffn1", EncoderLinear), ("ffn2", EncoderLinear),
                ("ffn1_out_scale", f32),
                ("ln1_gamma", c_p), ("ln1_beta", c_p), ("ln2_gamma", c_p), ("ln2_beta", c_p),
                ("s_x", f32), ("s_qkv", f32), ("s_ctx", f32), ("s_ao", f32), ("s_h", f32), ("s_f", f32), ("s_out", f32)]


class EncoderBatch(C.Structure):
    _fields_ = [("ids", c_p), ("segment_ids", c_p), ("cu_seqlens", c_p), ("batch", i32), ("tokens", i32),
                ("workspace", c_p), ("out", c_p)]


_SIGS = {
    "trtamd_version": (C.c_int, []),
    "trtamd_last_error": (C.c_char_p, []),
    "trtamd_skip_layer_norm_fp32": (C.c_int, [c_p, i32, i64, c_p, c_p, c_p, c_p, c_p, c_p]),
    "trtamd_skip_layer_norm_fp16": (C.c_int, [c_p, i32, i64, c_p, c_p, c_p, c_p, c_p, c_p]),
    "trtamd_skip_layer_norm_dqq": (C.c_int, [c_p, i32, i64, c_p, c_p, c_p, c_p, c_p, c_p, f32, f32, f32]),
    "trtamd_skipln_interleaved_small_hface": (C.c_int, [c_p, i32, i32, c_p, c_p, c_p, c_p, c_p, f32, f32, f32]),
    "trtamd_skipln_interleaved_large_hface": (C.c_int, [c_p, i32, i32, c_p, c_p, c_p, c_p, c_p, f32, f32, f32]),
    "trtamd_skipln_interleaved_small_mtron": (C.c_int, [c_p, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, f32, f32, f32,
                                                        f32]),
    "trtamd_skipln_interleaved_large_mtron": (C.c_int, [c_p, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, f32, f32, f32,
                                                        f32]),
    "trtamd_emb_layer_norm_fp32": (C.c_int, [c_p, i32, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, i32, i32, c_p]),
    "trtamd_emb_layer_norm_fp16": (C.c_int, [c_p, i32, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, i32, i32, c_p]),
    "trtamd_emb_layer_norm_hface_fp32": (C.c_int, [c_p, i32, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, i32, i32,
                                                   c_p]),
    "trtamd_emb_layer_norm_hface_fp16": (C.c_int, [c_p, i32, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, i32, i32,
                                                   c_p]),
    "trtamd_emb_layer_norm_mtron_fp32": (C.c_int, [c_p, i32, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, i32, i32,
                                                   c_p, c_p]),
    "trtamd_emb_layer_norm_mtron_fp16": (C.c_int, [c_p, i32, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, i32, i32,
                                                   c_p, c_p]),
    "trtamd_compute_mask_idx": (C.c_int, [c_p, i32, i32, c_p, c_p]),
    "trtamd_convert_mask": (C.c_int, [u32, u32, u32, u32, u32, c_p, c_p, c_p]),
    "trtamd_scaled_softmax_fp32": (C.c_int, [c_p, i32, i32, i32, f32, c_p, c_p, c_p]),
    "trtamd_scaled_softmax_fp16": (C.c_int, [c_p, i32, i32, i32, f32, c_p, c_p, c_p]),
    "trtamd_unfused_mha_workspace_size": (C.c_size_t, [i32, i32, i32, i32]),
    "trtamd_unfused_mha": (C.c_int, [c_p, i32, i32, i32, i32, i32, c_p, c_p, c_p, c_p]),
    "trtamd_unfused_mha_routed": (C.c_int, [c_p, i32, i32, i32, i32, i32, i32, c_p, c_p, c_p, c_p]),
    "trtamd_unfused_mha_tune": (C.c_int, [i32, i32, i32, i32, i32, C.POINTER(C.c_int32), C.POINTER(C.c_float)]),
    "trtamd_unfused_mha_static_capacity": (C.c_size_t, []),
    "trtamd_unfused_mha_static_prepare": (C.c_int, []),
    "trtamd_test_set_tuning": (C.c_int, [C.c_char_p, i32]),
    "trtamd_test_reset_tuning": (C.c_int, [C.c_char_p]),
    "trtamd_unfused_mha_static": (C.c_int, [c_p, i32, i32, i32, i32, i32, c_p, c_p, c_p]),
    "trtamd_fused_mha_run": (C.c_int, [c_p, i32, C.POINTER(FmhaParams)]),
    "trtamd_fused_mha_run_debug": (C.c_int, [c_p, i32, C.POINTER(FmhaParams), c_p, c_p]),
    "trtamd_fused_mha_prepare": (C.c_int, []),
    "trtamd_fused_mha_is_valid": (C.c_int, [i32, i32, i32]),
    "trtamd_zero_padding_2d": (C.c_int, [c_p, i32, c_p, i32, i32, c_p]),
    "trtamd_int8_linear": (C.c_int, [c_p, C.POINTER(Int8LinearParams)]),
    "trtamd_fp16_linear": (C.c_int, [c_p, C.POINTER(Fp16LinearParams)]),
    "trtamd_encoder_create": (c_p, [C.POINTER(EncoderConfig)]),
    "trtamd_encoder_destroy": (None, [c_p]),
    "trtamd_encoder_set_embedding": (C.c_int, [c_p, C.POINTER(EncoderEmbedding)]),
    "trtamd_encoder_set_layer": (C.c_int, [c_p, i32, C.POINTER(EncoderLayer)]),
    "trtamd_encoder_workspace_size": (C.c_size_t, [c_p, i32]),
    "trtamd_encoder_enqueue": (C.c_int, [c_p, c_p, c_p, c_p, i32, i32, c_p, c_p, c_p]),
    "trtamd_encoder_reserve_contexts": (C.c_int, [c_p, i32]),
    "trtamd_encoder_enqueue_concurrent": (C.c_int, [c_p, C.POINTER(EncoderBatch), i32, c_p]),
    "trtamd_int8_linear_to_interleaved": (C.c_int, [c_p, i32, i32, c_p, c_p]),
    "trtamd_int8_interleaved_to_linear": (C.c_int, [c_p, i32, i32, c_p, c_p]),
    "trtamd_quantize_fp16_to_interleaved": (C.c_int, [c_p, i32, i32, c_p, f32, c_p]),
    "trtamd_dequantize_interleaved_to_fp16": (C.c_int, [c_p, i32, i32, c_p, f32, c_p]),
}

# Entry points declared in include/trtamd_test_hooks.h (test-only).
TEST_HOOK_SYMBOLS = ["trtamd_fused_mha_run_debug", "trtamd_test_set_tuning", "trtamd_test_reset_tuning"]
# Entry points declared in include/trtamd_bert_kernels.h are the rest of the table.
# Entry points declared in include/trtamd_encoder_ops.h.
ENCODER_OPS_SYMBOLS = ["trtamd_int8_linear", "trtamd_fp16_linear", "trtamd_int8_linear_to_interleaved", "trtamd_int8_interleaved_to_linear",
                       "trtamd_quantize_fp16_to_interleaved", "trtamd_dequantize_interleaved_to_fp16"]
# Entry points declared in include/trtamd_encoder_runtime.h.
ENCODER_RUNTIME_SYMBOLS = ["trtamd_encoder_create", "trtamd_encoder_destroy", "trtamd_encoder_set_embedding",
                           "trtamd_encoder_set_layer", "trtamd_encoder_workspace_size", "trtamd_encoder_enqueue",
                           "trtamd_encoder_reserve_contexts", "trtamd_encoder_enqueue_concurrent"]
HEADER_SYMBOLS = [k for k in _SIGS if k not in TEST_HOOK_SYMBOLS and k not in ENCODER_OPS_SYMBOLS
                  and k not in ENCODER_RUNTIME_SYMBOLS]


class TrtAmdError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"status {status}: {message}")
        self.status = status
        self.message = message


class _Api:
    def __init__(self):
        self._lib = load_library()
        for name, (res, args) in _SIGS.items():
            fn = getattr(self._lib, name)
            fn.restype = res
            fn.argtypes = args
            setattr(self, name[len("trtamd_"):], fn)

    def last_error_str(self) -> str:
        return (self.last_error() or b"").decode()

    def check(self, status: int) -> None:
        if status != 0:
            raise TrtAmdError(status, self.last_error_str())


_api = None


def api() -> _Api:
    global _api
    if _api is None:
        _api = _Api()
    return _api
