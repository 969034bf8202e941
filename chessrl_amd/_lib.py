"""ctypes binding of include/chessrl_amd.h.

The library is loaded from chessrl_amd/libchessrl_amd.so (built in-tree by
``python -m chessrl_amd.build``). There is no fallback: if the shared object is
missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libchessrl_amd.so")


class CrlError(RuntimeError):
    pass


class ModelConfig(C.Structure):
    _fields_ = [
        ("arch", C.c_int32), ("n_layer", C.c_int32), ("d_model", C.c_int32), ("n_head", C.c_int32),
        ("d_ff", C.c_int32), ("fp8", C.c_int32), ("micro_batch", C.c_int32), ("stream_f32", C.c_int32),
        ("head_dtype", C.c_int32), ("smolgen_compress", C.c_int32), ("smolgen_hidden", C.c_int32),
        ("smolgen_gen", C.c_int32), ("eps", C.c_float), ("act_dtype", C.c_int32), ("ln_fold", C.c_int32), ("norm_rms", C.c_int32), ("fp8_lm_head", C.c_int32),
    ]


F32, BF16, F16, FP8 = 0, 1, 2, 3
ACT_NONE, ACT_GELU, ACT_MISH, ACT_SWISH = 0, 1, 2, 3
ATTN_PLAIN, ATTN_CAUSAL, ATTN_BIAS, ATTN_RELSHIFT = 0, 1, 2, 3
ARCH_GPT64, ARCH_BT4, ARCH_BT4CLASS = 0, 1, 2
VOCAB_RL, VOCAB_LEELA, NUM_PLANES = 1929, 1858, 19

_vp, _i, _i64, _f, _cp = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_char_p
_pp = C.POINTER(C.c_char_p)

# name -> (restype, argtypes); every symbol include/chessrl_amd.h declares.
SIGNATURES = {
    "crl_last_error": (_cp, []),
    "crl_version": (_cp, []),
    "crl_policy_index": (_cp, [_i]),
    "crl_policy_leela": (_cp, [_i]),
    "crl_move_to_index": (_i, [_cp]),
    "crl_leela_to_rl_maps": (_i, [_vp, _vp]),
    "crl_fen_to_planes": (_i, [_cp, _vp]),
    "crl_encode_fens": (_i, [_pp, _i, _vp, _i]),
    "crl_encode_fens_compact": (_i, [_pp, _i, _vp, _vp, _i]),
    "crl_legal_masks": (_i, [_pp, _i, _vp, _vp, _i]),
    "crl_legal_masks_leela": (_i, [_pp, _i, _vp, _vp, _i]),
    "crl_legal_moves": (_i, [_cp, _vp, _i]),
    "crl_child_fens": (_i, [_cp, _vp, _vp, _i]),
    "crl_perft": (C.c_uint64, [_cp, _i]),
    "crl_random_positions": (_i, [C.c_uint64, _i, _i, C.c_double, _i, _vp, _vp, _vp, _vp]),
    "crl_gemm": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _i, _vp, _i, _f, _f, _vp, _i64, _i, _f, _vp, _i, _vp]),
    "crl_gemm_split": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _i, _i, _vp, _f, _i, _vp]),
    "crl_gemm_static_scratch": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _i, _vp, _i, _f, _f, _vp, _i64, _i, _f, _vp, _vp]),
    "crl_gemm_static_scratch_bytes": (_i64, []),
    "crl_shutdown": (None, []),
    "crl_layernorm": (_i, [_vp, _i64, _i, _vp, _vp, _vp, _i, _vp, _f, _i64, _i, _i, _f, _vp, _vp]),
    "crl_rmsnorm": (_i, [_vp, _i64, _i, _vp, _vp, _i, _vp, _f, _i64, _i, _i, _f, _vp, _vp]),
    "crl_attention": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _i, _vp, _i64, _i, _f, _i, _i, _i, _i, _f, _vp, _vp, _vp, _vp, _vp, _vp]),
    "crl_attn_bias_slot": (_i, [_i, _i]),
    "crl_masked_softmax": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i, _i, _f, _vp]),
    "crl_leela_to_rl": (_i, [_vp, _i64, _vp, _i64, _vp, _i, _vp]),
    "crl_model_create": (_i, [C.POINTER(ModelConfig), C.POINTER(_vp)]),
    "crl_model_destroy": (None, [_vp]),
    "crl_model_set_weight": (_i, [_vp, _cp, _vp, _i64]),
    "crl_model_expected_key": (_cp, [_vp, _i, C.POINTER(_i64)]),
    "crl_model_finalize": (_i, [_vp]),
    "crl_model_calibrate": (_i, [_vp, _vp, _i, _vp]),
    "crl_model_get_amax": (_i, [_vp, _vp, _i]),
    "crl_model_set_amax": (_i, [_vp, _vp, _i]),
    "crl_model_forward": (_i, [_vp, _vp, _i, _vp, _vp, _vp]),
    "crl_model_forward_compact": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp]),
    "crl_model_run_layers": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "crl_model_read_tensor": (_i, [_vp, _cp, _vp, _i64, _vp]),
    "crl_model_vocab": (_i, [_vp]),
    "crl_model_flops_per_position": (C.c_double, [_vp]),
    "crl_model_set_profiling": (_i, [_vp, _i]),
    "crl_model_set_decode_graph": (_i, [_vp, _i]),
    "crl_model_get_profile": (_i, [_vp, _vp, _vp, _vp]),
    "crl_model_evaluate_fens": (_i, [_vp, C.POINTER(C.c_char_p), _i, _i, _f, _vp, _vp, _vp, _i]),
    "crl_model_search_1ply": (_i, [_vp, C.POINTER(C.c_char_p), _i, _i, _f, C.c_uint64, _vp, _vp, _vp, _vp, _i64, _i]),
    "crl_model_forward_tokens": (_i, [_vp, _vp, _vp, _i, _i, _vp, _vp, _vp]),
    "crl_attention_causal": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _i, _vp, _i64, _i, _f, _i, _i, _i, _i, _f, _vp, _vp]),
    "crl_token_scores": (_i, [_vp, _i64, _vp, _i64, _vp, _i, _i, _i64, _vp, _vp, _vp, _vp]),
    "crl_masked_nll_mean": (_i, [_vp, _vp, _i64, _i, _vp, _vp]),
    "crl_model_generate": (_i, [_vp, _vp, _i, _i, _f, C.c_uint64, _i, _vp, _vp, _i, _vp]),
    "crl_sample": (_i, [_vp, _i64, _i, _i, _f, C.c_uint64, _i, _vp, _vp, _vp]),
    "crl_probe_mfma": (_i, [_i, _i, _i, _vp, _vp, _vp]),
    "crl_probe_cu_split": (_i, [_i, _i, _i, _i, _vp]),
}

_lib = None


def lib():
    """The loaded shared library (raises CrlError when it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CrlError("%s is missing: run `python -m chessrl_amd.build` (hipcc, gfx950)" % LIB_PATH)
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc, what=""):
    """Raise CrlError for a negative return code."""
    if rc is not None and rc < 0:
        msg = lib().crl_last_error()
        raise CrlError("%s failed (%d): %s" % (what or "chessrl_amd call", rc, msg.decode() if msg else ""))
    return rc


def str_array(strings):
    arr = (C.c_char_p * len(strings))()
    arr[:] = [s.encode() if isinstance(s, str) else s for s in strings]
    return arr
