"""ctypes bindings of libffmoe.so. Every function takes raw device addresses (ints) and sizes.

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# FFMOE_LIBRARY names another build of the same library (A/B measurements of two builds in one session)
LIB_PATH = os.environ.get("FFMOE_LIBRARY") or os.path.join(_HERE, "libffmoe.so")

# enums of include/ffmoe.h
FMT_FP8_BLOCK128, FMT_NVFP4, FMT_BF16, FMT_FP8_CHANNEL, FMT_E2M1_E8M0, FMT_E4M3_E8M0_32 = 0, 1, 2, 3, 4, 5
FORM_LANE16, FORM_LANE8 = 0, 1
ACT_BF16, ACT_FP8_BLOCK128, ACT_E4M3_E8M0_32, ACT_E4M3_E8M0_32_F32 = 0, 1, 2, 3
SWIGLU_TWICE, SWIGLU_ONCE, SWIGLU_CLAMPED_TWICE, SWIGLU_CLAMPED_ONCE, SWIGLU_GELU_TWICE = 0, 1, 2, 3, 4
WEIGHT_AFTER_DOWN_BF16, WEIGHT_BEFORE_CONTRIBUTION_BF16, WEIGHT_BEFORE_DOWN_F32 = 0, 1, 2
SCORE_SOFTMAX, SCORE_SIGMOID = 0, 1
NOAUX_SIGMOID, NOAUX_SQRTSOFTPLUS = 0, 1
COMBINE_GATED, COMBINE_UNGATED, COMBINE_BF16, COMBINE_ACCUM_FP32, COMBINE_ACCUM_BF16, COMBINE_ROUTED = range(6)
ERR_NULL, ERR_ALIGN, ERR_SHAPE, ERR_OVERLAP, ERR_UNSUPPORTED, ERR_SCRATCH = -1, -2, -3, -4, -5, -6

EXPORTS = [
    "ffmoe_last_error", "ffmoe_version",
    "ffmoe_route_logits_bf16", "ffmoe_route_logits_f32", "ffmoe_route_topk", "ffmoe_route_topk_noaux", "ffmoe_route_noaux_decode", "ffmoe_route_decode", "ffmoe_slot_publish", "ffmoe_route_mask",
    "ffmoe_decode_scratch_bytes", "ffmoe_decode_contribute", "ffmoe_decode_static_scratch_bytes", "ffmoe_decode_contribute_static", "ffmoe_decode_contribute_stage", "ffmoe_decode_finish", "ffmoe_decode_contribute_from_logits", "ffmoe_decode_token_layer", "ffmoe_decode_token_forward", "ffmoe_decode_token_forward_stage", "ffmoe_decode_contribute_form", "ffmoe_e8m0_scratch_bytes", "ffmoe_decode_contribute_e8m0", "ffmoe_act_quant_e8m0",
    "ffmoe_quant_fp8_f32_128", "ffmoe_linear_fp8_block_w8a8", "ffmoe_linear_fp8_block", "ffmoe_linear_fp8_block_batch", "ffmoe_linear_nvfp4",
    "ffmoe_gemm_skinny_bf16", "ffmoe_swiglu",
    "ffmoe_shared_scale", "ffmoe_combine",
    "ffmoe_combine_residual", "ffmoe_prefill_scratch_bytes", "ffmoe_prefill_contribute", "ffmoe_prefill_contribute_stage",
]

P = ctypes.c_void_p
I = ctypes.c_int
F = ctypes.c_float
U64 = ctypes.c_uint64


class ExpertTable(ctypes.Structure):
    _fields_ = [("format", I), ("experts", I), ("hidden", I), ("inter", I),
                ("slots", P), ("valid", P), ("global_scales", P), ("generation", P)]


class SharedExpert(ctypes.Structure):
    _fields_ = [("format", I), ("inter", I), ("slot", U64 * 6), ("global_scales", F * 3)]


class Decode(ctypes.Structure):
    _fields_ = [("rows", I), ("top_k", I), ("act_mode", I), ("swiglu", I), ("swiglu_limit", F),
                ("routed_weight", I), ("weights_f32", I),
                ("x", P), ("ids", P), ("active", P), ("weights", P),
                ("contributions", P), ("shared_out", P), ("done", P),
                ("scratch", P), ("scratch_bytes", U64), ("assignment_gen", P)]


class Prefill(ctypes.Structure):
    _fields_ = [("rows", I), ("top_k", I), ("act_mode", I), ("swiglu", I), ("swiglu_limit", F), ("routed_weight", I),
                ("weights_f32", I), ("x", P), ("ids", P), ("active", P), ("weights", P),
                ("contributions", P), ("done", P), ("scratch", P), ("scratch_bytes", U64),
                ("shared", ctypes.POINTER(SharedExpert)), ("shared_out", P), ("assignment_gen", P)]


class FfmoeError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("libffmoe error %d: %s" % (code, text))
        self.code = code


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libffmoe.so is not built (%s); run `python -m flyingfish_amd.build`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.ffmoe_last_error.restype = ctypes.c_char_p
        L.ffmoe_version.restype = I
        L.ffmoe_route_logits_bf16.argtypes = [P, P, P, I, I, I, P]
        L.ffmoe_route_logits_f32.argtypes = [P, P, P, I, I, I, P]
        L.ffmoe_route_topk.argtypes = [P, P, P, I, I, I, I, P]
        L.ffmoe_route_topk_noaux.argtypes = [P, P, I, P, P, I, I, I, I, I, F, I, I, P]
        L.ffmoe_route_noaux_decode.argtypes = [P, P, P, I, P, P, P, I, P, I, I, I, I, I, F, I, I, P]
        L.ffmoe_route_decode.argtypes = [P, P, P, P, P, I, I, I, I, I, P]
        L.ffmoe_slot_publish.argtypes = [P, P, P, I, I, I, ctypes.POINTER(U64 * 6), U64, P, P]
        L.ffmoe_route_mask.argtypes = [P, P, P, P, P, P, I, I, P]
        L.ffmoe_decode_scratch_bytes.restype = U64
        L.ffmoe_decode_scratch_bytes.argtypes = [I, I, I, I, I, I]
        L.ffmoe_decode_contribute.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode), P]
        L.ffmoe_decode_static_scratch_bytes.restype = U64
        L.ffmoe_decode_static_scratch_bytes.argtypes = []
        L.ffmoe_decode_contribute_static.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode), P]
        L.ffmoe_decode_contribute_stage.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode), I, P]
        L.ffmoe_quant_fp8_f32_128.argtypes = [P, P, P, I, I, P]
        L.ffmoe_linear_fp8_block_w8a8.argtypes = [P, P, P, P, P, I, I, I, P]
        L.ffmoe_linear_fp8_block.argtypes = [P, P, P, P, I, I, I, I, P, U64, P]
        L.ffmoe_linear_fp8_block_batch.argtypes = [P, I, I, I, I, P]
        L.ffmoe_linear_nvfp4.argtypes = [P, P, P, P, P, I, I, I, P]
        L.ffmoe_gemm_skinny_bf16.argtypes = [P, P, P, I, I, I, P]
        L.ffmoe_swiglu.argtypes = [P, P, P, I, I, I, F, P]
        L.ffmoe_shared_scale.argtypes = [P, P, P, I, I, P]
        L.ffmoe_combine.argtypes = [P, P, P, P, P, P, P, P, I, I, I, I, P]
        L.ffmoe_decode_contribute_from_logits.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode),
                                                          P, P, I, F, I, I, P]
        L.ffmoe_decode_token_layer.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode),
                                               P, P, I, F, I, I, P, P, P, I, P]
        L.ffmoe_decode_token_forward.argtypes = L.ffmoe_decode_token_layer.argtypes
        L.ffmoe_decode_token_forward_stage.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode),
                                                       P, P, I, F, I, I, P, P, P, I, I, P]
        L.ffmoe_decode_contribute_form.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode), I, P]
        L.ffmoe_e8m0_scratch_bytes.restype = ctypes.c_uint64
        L.ffmoe_e8m0_scratch_bytes.argtypes = [I, I, I, I, I]
        L.ffmoe_decode_contribute_e8m0.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode), P]
        L.ffmoe_act_quant_e8m0.argtypes = [P, P, P, I, I, P]
        L.ffmoe_decode_finish.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(SharedExpert), ctypes.POINTER(Decode), P, P, P, I, P]
        L.ffmoe_combine_residual.argtypes = [P, P, P, P, P, ctypes.c_longlong, P, P, P, P, P, P, I, I, I, P]
        L.ffmoe_prefill_scratch_bytes.restype = U64
        L.ffmoe_prefill_scratch_bytes.argtypes = [I, I, I, I, I, I]
        L.ffmoe_prefill_contribute.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(Prefill), P]
        L.ffmoe_prefill_contribute_stage.argtypes = [ctypes.POINTER(ExpertTable), ctypes.POINTER(Prefill), I, P]
        for name in EXPORTS:
            fn = getattr(L, name)
            if fn.restype is ctypes.c_int or name not in ("ffmoe_last_error", "ffmoe_decode_scratch_bytes", "ffmoe_prefill_scratch_bytes"):
                fn.restype = fn.restype if name in ("ffmoe_last_error",) else (U64 if "scratch_bytes" in name else I)
        _lib = L
    return _lib


def check(code):
    """Raise FfmoeError unless code == 0."""
    if code != 0:
        raise FfmoeError(code, lib().ffmoe_last_error().decode())
    return code


def last_error():
    return lib().ffmoe_last_error().decode()
