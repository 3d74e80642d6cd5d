"""ctypes binding of libet_hip.so (the C ABI declared in include/et.h).

The library is the product: if it is missing or does not load, importing callers get an
ImportError -- there is no fallback implementation.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libet_hip.so")

ET_OK = 0
ET_FP32, ET_FP16 = 0, 1
STATUS_NAMES = {0: "ET_OK", 1: "ET_INVALID_ARGUMENT", 2: "ET_WORKSPACE_TOO_SMALL", 3: "ET_UNSUPPORTED",
                4: "ET_LAUNCH_FAILURE", 5: "ET_RUNTIME_ERROR"}

WEIGHT_FIELDS = (
    "attr_kernel_Q", "attr_kernel_K", "attr_kernel_V", "attr_bias_Q", "attr_bias_K", "attr_bias_V",
    "attr_output_kernel", "attr_output_bias", "attr_output_layernorm_gamma", "attr_output_layernorm_beta",
    "inter_kernel", "inter_bias", "output_kernel", "output_bias", "output_layernorm_gamma",
    "output_layernorm_beta",
)


class LayerWeights(C.Structure):
    _fields_ = [(name, C.c_void_p) for name in WEIGHT_FIELDS]


class LayerPrepared(C.Structure):
    _fields_ = [("attr_kernel_Q_t", C.c_void_p), ("attr_kernel_K_t", C.c_void_p), ("attr_kernel_V_t", C.c_void_p),
                ("attr_output_kernel_t", C.c_void_p), ("inter_kernel_t", C.c_void_p), ("output_kernel_t", C.c_void_p),
                ("seq_start", C.c_void_p), ("warm", C.c_void_p), ("warm_bytes", C.c_size_t),
                ("seq_start_bytes", C.c_size_t)]


class EmbeddingWeights(C.Structure):
    _fields_ = [("word_embeddings", C.c_void_p), ("token_type_embeddings", C.c_void_p),
                ("position_embeddings", C.c_void_p), ("layernorm_gamma", C.c_void_p), ("layernorm_beta", C.c_void_p),
                ("vocab_size", C.c_int), ("type_vocab_size", C.c_int), ("max_position_embeddings", C.c_int)]


class EtError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__("%s: %s" % (STATUS_NAMES.get(status, str(status)), message))
        self.status = status


_vp, _i, _sz, _ip = C.c_void_p, C.c_int, C.c_size_t, C.POINTER(C.c_int32)

# name -> (restype, argtypes); every symbol include/et.h declares
SIGNATURES = {
    "et_create": (_i, [C.POINTER(_vp), _i]),
    "et_destroy": (_i, [_vp]),
    "et_last_error": (C.c_char_p, [_vp]),
    "et_status_string": (C.c_char_p, [_i]),
    "et_device_ok": (_i, [_i]),
    "et_input_workspace_bytes": (_sz, [_i, _i]),
    "et_layer_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "et_seq_workspace_bytes": (_sz, [_i]),
    "et_input": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _sz, _vp, _ip]),
    "et_input_static": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "et_embedding_input": (_i, [_vp, _i, C.POINTER(EmbeddingWeights), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i,
                                _vp, _sz, _vp, _ip]),
    "et_layer": (_i, [_vp, _i, C.POINTER(LayerWeights), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i,
                      _vp, _sz, _vp]),
    "et_sequence_starts": (_i, [_vp, _vp, _vp, _i, _i, _vp, _sz, _vp]),
    "et_layer_with_prepared": (_i, [_vp, _i, C.POINTER(LayerWeights), C.POINTER(LayerPrepared), _vp, _vp, _vp, _vp, _vp,
                                    _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "et_first_token": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "et_output": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "et_exclusive_scan": (_i, [_vp, _vp, _vp, _i, _vp, _sz, _vp]),
    "et_compress": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "et_restore": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "et_add_bias_act": (_i, [_vp, _i, _vp, _vp, _i, _i, _vp, _vp]),
    "et_add_bias_input_layernorm": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "et_add_qkv_bias_padding": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i,
                                     _vp, _vp, _vp, _sz, _vp]),
    "et_softmax": (_i, [_vp, _i, _vp, _vp, _i, _i, _i, C.c_float, _vp]),
    "et_transpose_rm_padding": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "et_attention": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _sz, _vp]),
    "et_attention_with_starts": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp,
                                      _sz, _vp]),
    "et_gemm": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "et_gemm_bias_gelu": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "et_transpose_weight": (_i, [_vp, _i, _vp, _vp, _i, _i, _vp]),
    "et_gemm_bt": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "et_gemm_bt_bias_gelu": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "et_calibrate_mfma_sink_bytes": (_sz, [_vp]),
    "et_calibrate_mfma": (_i, [_vp, _i, _i, _vp, _sz, C.POINTER(C.c_double), _vp]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the library (once).  Raises ImportError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libet_hip.so is not built (%s); run `python -m effective_transformer_amd.build`" % LIB_PATH)
    try:
        lib = C.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise ImportError("libet_hip.so failed to load: %s" % e) from e
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)       # AttributeError here means the header and the library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, handle=None) -> None:
    if status != ET_OK:
        msg = load().et_last_error(handle)
        raise EtError(status, msg.decode() if msg else "")
