"""ctypes binding of libvui_amd.so (the C ABI declared in include/vui_amd.h).

The library is loaded from the package directory; there is no fallback: if it is missing or a
call fails, a RuntimeError carrying vui_last_error() is raised.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libvui_amd.so")

VUI_MAX_LAYERS = 64
VUI_MAX_RQ_LAYERS = 16
VUI_MAX_BATCH = 16
DTYPE_BF16, DTYPE_F32 = 0, 1


class VuiConfigC(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "dtype", "d_model", "n_layers", "n_heads", "n_kv_heads", "head_dim", "ffn", "n_quantizers",
        "codebook_size", "rq_dim", "rq_layers", "rq_heads", "rq_ffn", "rope_dim", "max_seqlen", "n_slots",
        "window")] + [("norm_eps", C.c_float), ("rq_norm_eps", C.c_float), ("int8_backbone", C.c_int32),
                      ("global_layers", C.c_uint64), ("global_rope_dim", C.c_int32), ("reserved", C.c_int32)]


class LayerWeightsC(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "attn_norm", "wqkv", "wo", "mlp_norm", "w1", "w3", "w2", "s_qkv", "s_o", "s_1", "s_3", "s_2")]


class RqLayerWeightsC(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("attn_norm", "wqkv", "wo", "mlp_norm", "w1", "w3", "w2")]


class WeightsC(C.Structure):
    _fields_ = [
        ("audio_emb", C.c_void_p), ("final_norm", C.c_void_p), ("codec_head", C.c_void_p),
        ("eos_w", C.c_void_p), ("eos_b", C.c_void_p), ("rope_table", C.c_void_p),
        ("layers", LayerWeightsC * VUI_MAX_LAYERS),
        ("rq_backbone_proj", C.c_void_p), ("rq_code_emb", C.c_void_p), ("rq_pos_emb", C.c_void_p),
        ("rq_head_w", C.c_void_p), ("rq_norm", C.c_void_p),
        ("rq_layers", RqLayerWeightsC * VUI_MAX_RQ_LAYERS),
        ("rope_table_global", C.c_void_p),
    ]


class SampleParamsC(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_int32), ("seed", C.c_uint64),
                ("frame_ctr", C.c_void_p), ("state_rows", C.c_void_p), ("keep_ties", C.c_int32), ("top_p", C.c_float), ("dev", C.c_void_p)]


class EosStopC(C.Structure):
    """vui_eos_stop (include/vui_amd.h)."""
    _fields_ = [("threshold", C.c_float), ("min_frames", C.c_int32), ("state", C.c_void_p)]


class CodecConfigC(C.Structure):
    """vui_codec_config (include/vui_codec.h)."""
    _fields_ = [(n, C.c_int32) for n in (
        "n_codebooks", "codebook_size", "codebook_dim", "vq_dim", "n_semantic", "latent_dim", "d_model", "n_layers",
        "n_heads", "head_dim", "mlp_dim", "max_seq")] + [
        ("rope_theta", C.c_float), ("n_up", C.c_int32), ("up_ratios", C.c_int32 * 4), ("decoder_dim", C.c_int32),
        ("n_rates", C.c_int32), ("rates", C.c_int32 * 8)]


# name -> (restype, argtypes); every symbol include/*.h declares
_P, _I, _L, _F = C.c_void_p, C.c_int, C.c_int64, C.c_float
SIGNATURES = {
    "vui_last_error": (C.c_char_p, []),
    "vui_version": (_I, []),
    "vui_workspace_bytes": (_L, [C.POINTER(VuiConfigC), _I]),
    "vui_kv_bytes": (_L, [C.POINTER(VuiConfigC)]),
    "vui_ctx_create": (_I, [C.POINTER(VuiConfigC), C.POINTER(WeightsC), _P, _L, _I, C.POINTER(_P)]),
    "vui_ctx_destroy": (None, [_P]),
    "vui_ctx_init": (_I, [_P, _P]),
    "vui_ctx_fused": (_I, [_P, _I]),
    "vui_ctx_status": (_I, [_P]),
    "vui_debug_set_epoch": (_I, [_P, C.c_uint32]),
    "vui_ctx_rq_batch": (_I, [_P]),
    "vui_ctx_bb_batch": (_I, [_P]),
    "vui_cu_stream_create": (_I, [_I, _I, C.POINTER(_P)]),
    "vui_ctx_workgroups": (_I, [_P, _I]),
    "vui_debug_phase_clock": (_I, [_P, _P, _I, _I]),
    "vui_prefill_scratch_bytes": (_L, [C.POINTER(VuiConfigC), _I, _I]),
    "vui_prefill": (_I, [_P, _P, _I, _I, _I, _P, _P, _P, _P, _P, _L, _P]),
    "vui_codec_hop": (C.c_int32, [C.POINTER(CodecConfigC)]),
    "vui_codec_n_tensors": (C.c_int32, [C.POINTER(CodecConfigC)]),
    "vui_codec_workspace_bytes": (_L, [C.POINTER(CodecConfigC)]),
    "vui_codec_init": (_I, [C.POINTER(CodecConfigC), C.POINTER(_P), C.c_int32, _P, _L, _P, C.POINTER(_P)]),
    "vui_codec_destroy": (None, [_P]),
    "vui_codec_reset": (_I, [_P, _P]),
    "vui_codec_decode_frame": (_I, [_P, _P, C.c_int32, _P, _P]),
    "vui_codec_status": (_L, [_P, _P]),
    "vui_codec_persistent": (_I, [_P, _I]),
    "vui_codec_workgroups": (_I, [_P, _I]),
    "vui_backbone_step": (_I, [_P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _P]),
    "vui_sample_cb0": (_I, [_P, _P, _P, _P, _P, _F, _I, C.POINTER(SampleParamsC), _P, _I, _P]),
    "vui_rq_generate": (_I, [_P, _P, _P, _P, _I, C.POINTER(SampleParamsC), _P, _I, _I, _I, _P]),
    "vui_frame_step": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _F, _I, C.POINTER(SampleParamsC),
                            C.POINTER(SampleParamsC), _P, _I, _P, _P, _P, _P, _I, _P, _I, C.POINTER(EosStopC), _P]),
    "vui_graph_begin": (_I, [_P]),
    "vui_graph_end": (_I, [_P, C.POINTER(_P)]),
    "vui_graph_launch": (_I, [_P, _P]),
    "vui_graph_destroy": (None, [_P]),
    "vui_rmsnorm_gemv": (_I, [_I, _P, _P, _F, _P, _P, _I, _P, _I, _I, _I, _P]),
    "vui_rope": (_I, [_I, _P, _P, _P, _I, _I, _I, _I, _P]),
    "vui_attn_scratch_bytes": (_L, [_I, _I, _I, _I]),
    "vui_decode_attn": (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P]),
    "vui_decode_attn_noalloc": (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]),
    "vui_sample_logits": (_I, [_P, _P, _I, C.POINTER(SampleParamsC), _I, _P, _I, _P]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the shared library (once) and types its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m vui_amd.build` (there is no fallback path)")
    # one HIP runtime per process: PyTorch brings its own copy, so it is loaded first and the library binds
    # to that one (loaded the other way round, kernels launched from here find no device)
    import torch  # noqa: F401

    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error() -> str:
    return load().vui_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed ({rc}): {last_error()}")


def ptr(t) -> int | None:
    """Device (or host) address of a torch tensor, None for None."""
    return None if t is None else t.data_ptr()
