"""ctypes binding of ``libgptoss_mi355.so`` (the C ABI in ``include/gptoss_mi355.h``).

The library is loaded from this directory; a missing library is an error (there is no CPU or
PyTorch fallback for any entry point)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libgptoss_mi355.so")

OK = 0
ERR_NAMES = {1: "GPTOSS_ERR_NULL", 2: "GPTOSS_ERR_DIM", 3: "GPTOSS_ERR_ALIGN",
             4: "GPTOSS_ERR_WORKSPACE", 5: "GPTOSS_ERR_HIP", 6: "GPTOSS_ERR_STATE",
             7: "GPTOSS_ERR_IO"}

PACK_SRC_FP32 = 1
PACK_GLU = 2
ENGINE_SYNTHETIC = 1
ENGINE_PRECISE = 2
ENGINE_LOGITS = 4
ENGINE_NO_PREFILL = 8
ENGINE_MXFP4_EXPERTS = 16


#: GPTOSS_TENSOR_* of gptoss_engine_tensor_view, in the header's order
TENSORS = ("embedding", "unembedding", "final_norm", "attn_norm", "mlp_norm", "qkv_weight", "qkv_bias",
           "out_weight", "out_bias", "sinks", "gate_weight", "gate_bias", "mlp1_weight", "mlp1_bias",
           "mlp2_weight", "mlp2_bias")


class GptossError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"{ERR_NAMES.get(code, code)}: {msg}")
        self.code = code


class MoeWeights(C.Structure):
    _fields_ = [("n_experts", C.c_int), ("top_k", C.c_int), ("hidden", C.c_int),
                ("intermediate", C.c_int), ("swiglu_limit", C.c_float),
                ("w_router", C.c_void_p), ("b_router", C.c_void_p), ("w1", C.c_void_p),
                ("b1", C.c_void_p), ("w2", C.c_void_p), ("b2", C.c_void_p)]


class Config(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("vocab_size", "hidden_dim", "n_experts",
                                       "experts_per_token", "intermediate_dim", "n_layers",
                                       "head_dim", "n_attn_heads", "n_kv_heads", "seq_len",
                                       "initial_context_length")] + \
               [("rope_theta", C.c_float), ("rope_scaling_factor", C.c_float),
                ("sliding_window", C.c_int), ("swiglu_limit", C.c_float)]

    @classmethod
    def from_config(cls, c):
        return cls(*[getattr(c, n) for n, _ in cls._fields_])


_vp, _i, _sz, _f = C.c_void_p, C.c_int, C.c_size_t, C.c_float

#: name -> (restype, argtypes); every symbol declared in include/gptoss_mi355.h
SIGNATURES = {
    "gptoss_last_error_string": (C.c_char_p, []),
    "gptoss_abi_version": (_i, []),
    "gptoss_trace_set": (_i, [_vp, _vp, _i]),
    "gptoss_trace_count": (_i, []),
    "gptoss_trace_name": (C.c_char_p, [_i]),
    "gptoss_packed_weight_bytes": (_sz, [_i, _i, _i]),
    "gptoss_pack_weight": (_i, [_vp, _vp, _i, _i, _i, _i, _vp]),
    "gptoss_router_gemm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "gptoss_moe_max_tiles": (_i, [_i, _i, _i, _i]),
    "gptoss_moe_route": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "gptoss_moe_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "gptoss_moe_forward": (_i, [C.POINTER(MoeWeights), _vp, _i, _vp, _i, _vp, _sz, _vp]),
    "gptoss_moe_workspace_views": (_i, [_vp, _i, _i, _i, _i, _i] + [C.POINTER(_vp)] * 6),
    "gptoss_packed_mxfp4_bytes": (_sz, [_i, _i, _i]),
    "gptoss_pack_mxfp4": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "gptoss_moe_forward_mxfp4": (_i, [C.POINTER(MoeWeights), _vp, _i, _vp, _i, _vp, _sz, _vp]),
    "gptoss_kv_cache_bytes": (_sz, [_i, _i, _i, _i]),
    "gptoss_kv_cache_write": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "gptoss_attn_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "gptoss_attn_decode": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "gptoss_attn_decode_static_max_bytes": (_sz, []),
    "gptoss_attn_decode_static": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "gptoss_embedding": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "gptoss_rmsnorm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "gptoss_dense_gemm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "gptoss_classifier_argmax_workspace_bytes": (_sz, [_i, _i]),
    "gptoss_classifier_argmax": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _sz, _vp]),
    "gptoss_argmax": (_i, [_vp, _vp, _i, _i, _vp]),
    "gptoss_rope_tables": (_i, [C.POINTER(Config), _i, _vp, _vp]),
    "gptoss_rope_kv_store": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "gptoss_engine_create": (_i, [C.POINTER(Config), _vp, _i, _i, _i, C.c_uint64,
                                  C.POINTER(_vp)]),
    "gptoss_engine_step": (_i, [_vp, _vp, _i, _i, _vp]),
    "gptoss_engine_prefill": (_i, [_vp, _vp, _i, _i, _vp]),
    "gptoss_engine_step_ragged": (_i, [_vp, _vp, _vp, _i, _vp]),
    "gptoss_engine_step_rows": (_i, [_vp, _i, _vp, _vp, _vp, _i, _vp, _vp]),
    "gptoss_engine_generate_ragged": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _vp, C.POINTER(C.c_longlong)]),
    "gptoss_attn_prefill_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "gptoss_attn_prefill": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "gptoss_engine_generate": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, C.POINTER(C.c_longlong)]),
    "gptoss_engine_destroy": (None, [_vp]),
    "gptoss_engine_tensor_view": (_i, [_vp, _i, _i, C.POINTER(_vp), C.POINTER(_sz)]),
    "gptoss_engine_debug_views": (_i, [_vp, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_sz)]),
    "gptoss_diag_mfma_rate": (_i, [_i, _i, _i, _vp, C.POINTER(C.c_double), _vp]),
}

_lib = None


def load(strict: bool = os.environ.get("GPTOSS_PARTIAL_LIB") != "1"):
    """Load the shared library and bind every declared entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with "
                          f"`python {os.path.join(HERE, 'build.py')}` (hipcc, gfx950)")
    L = C.CDLL(LIB_PATH)
    missing = []
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(L, name)
        except AttributeError:
            missing.append(name)
            continue
        fn.restype = res
        fn.argtypes = args
    if missing and strict:
        raise ImportError(f"{LIB_PATH} does not export: {', '.join(missing)}")
    _lib = L
    return L


def last_error() -> str:
    return load().gptoss_last_error_string().decode()


def check(rc: int) -> None:
    if rc != OK:
        raise GptossError(rc, last_error())
