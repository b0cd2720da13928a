"""ctypes/numpy front end of the CPU oracle (``libgptoss_oracle.so``) and, when it has been
built, of the compiled reference CPU model (``_ref/libref_run.so``).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.  The shipped library never loads it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libgptoss_oracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libref_run.so")

STAGE_NORM, STAGE_KV, STAGE_ATTN, STAGE_SWIGLU, STAGE_Q, STAGE_FLOAT_ACC = 1, 2, 4, 8, 16, 32
#: rounding points of the reference GPU dataflow (bf16 activations into every GEMM)
STAGE_GPU = STAGE_NORM | STAGE_KV | STAGE_ATTN | STAGE_SWIGLU


class OrcConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("vocab_size", "hidden_dim", "n_experts",
                                       "experts_per_token", "intermediate_dim", "n_layers",
                                       "head_dim", "n_attn_heads", "n_kv_heads", "seq_len",
                                       "initial_context_length")] + \
               [("rope_theta", C.c_float), ("rope_scaling_factor", C.c_float),
                ("sliding_window", C.c_int), ("swiglu_limit", C.c_float)]

    @classmethod
    def from_config(cls, c):
        return cls(*[getattr(c, n) for n, _ in cls._fields_])


def build(ref: bool = True) -> None:
    """Compile the oracle (and the reference CPU model when /root/reference is present)."""
    subprocess.run(["make", "-s", "-B", "libgptoss_oracle.so"], cwd=HERE, check=True)
    if ref and os.path.exists("/root/reference/run.cpp"):
        subprocess.run(["make", "-s", "-B", "ref"], cwd=HERE, check=True)
        # the reference's run executable around this repository's getp hooks (needs the product library)
        pkg = os.path.join(os.path.dirname(HERE), "gpt-oss-team01_amd", "libgptoss_mi355.so")
        if os.path.exists(pkg):
            subprocess.run(["make", "-s", "-B", "getp"], cwd=HERE, check=True)


_lib = None
_ref = None


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build(ref=False)
        L = C.CDLL(LIB_PATH)
        L.orc_weight_floats.restype = C.c_longlong
        L.orc_generate.restype = C.c_longlong
        L.orc_model_create.restype = C.c_void_p
        L.orc_forward.restype = C.POINTER(C.c_float)
        L.orc_model_x.restype = C.POINTER(C.c_float)
        L.orc_model_last_router_gap.restype = C.c_float
        L.orc_model_min_router_gap.restype = C.c_float
        _lib = L
    return _lib


def have_ref() -> bool:
    return os.path.exists(REF_PATH)


def ref():
    global _ref
    if _ref is None:
        R = C.CDLL(REF_PATH)
        R.ref_open.restype = C.c_void_p
        R.ref_forward.restype = C.POINTER(C.c_float)
        R.ref_state_x.restype = C.POINTER(C.c_float)
        R.ref_generate.restype = C.c_longlong
        _ref = R
    return _ref


def num_threads() -> int:
    return int(lib().orc_num_threads())


# --------------------------------------------------------------------------- small ops
def rmsnorm(x, w):
    x, w = _f32(x), _f32(w)
    o = np.empty_like(x)
    lib().orc_rmsnorm(_fp(o), _fp(x), _fp(w), C.c_int(x.size))
    return o


def softmax(x):
    x = _f32(x).copy()
    lib().orc_softmax(_fp(x), C.c_int(x.size))
    return x


def matmul(x, w):
    x, w = _f32(x), _f32(w)
    d, n = w.shape
    o = np.empty(d, np.float32)
    lib().orc_matmul(_fp(o), _fp(x), _fp(w), C.c_int(n), C.c_int(d))
    return o


def topk_softmax(logits, k):
    logits = _f32(logits)
    B, E = logits.shape
    v = np.empty((B, k), np.float32)
    i = np.empty((B, k), np.int32)
    lib().orc_topk_softmax(_fp(logits), C.c_int(B), C.c_int(E), C.c_int(k), _fp(v), _ip(i))
    return v, i


def group(topk_i, E):
    topk_i = _i32(topk_i)
    B, k = topk_i.shape
    off = np.empty(E + 1, np.int32)
    srt = np.full(B * k, -1, np.int32)
    inv = np.full(B * k, -1, np.int32)
    lib().orc_group(_ip(topk_i), C.c_int(B), C.c_int(k), C.c_int(E), _ip(off), _ip(srt), _ip(inv))
    return off, srt, inv


def swiglu(mlp1_out, limit=7.0):
    m = _f32(mlp1_out)
    rows = m.reshape(-1, m.shape[-1])
    I = rows.shape[1] // 2
    out = np.empty((rows.shape[0], I), np.float32)
    for r in range(rows.shape[0]):
        lib().orc_swiglu(_fp(rows[r]), _fp(out[r]), C.c_int(I), C.c_float(limit))
    return out.reshape(m.shape[:-1] + (I,))


def moe_layer(t, w_router, b_router, w1, b1, w2, b2, k=4, limit=7.0, stage=0, want_routing=False):
    """t [B,H]; w_router [E,H]; w1 [E,2I,H]; w2 [E,H,I] -> e_agg [B,H] (fp32)."""
    t, w_router, b_router = _f32(t), _f32(w_router), _f32(b_router)
    w1, b1, w2, b2 = _f32(w1), _f32(b1), _f32(w2), _f32(b2)
    B, H = t.shape
    E = w_router.shape[0]
    I = w2.shape[2]
    assert w1.shape == (E, 2 * I, H) and w2.shape == (E, H, I)
    out = np.empty((B, H), np.float32)
    logits = np.empty((B, E), np.float32)
    tv = np.empty((B, k), np.float32)
    ti = np.empty((B, k), np.int32)
    lib().orc_moe_layer(_fp(t), _fp(w_router), _fp(b_router), _fp(w1), _fp(b1), _fp(w2), _fp(b2),
                        C.c_int(B), C.c_int(H), C.c_int(I), C.c_int(E), C.c_int(k),
                        C.c_float(limit), C.c_int(stage), _fp(out), _fp(logits), _fp(tv), _ip(ti))
    if want_routing:
        return out, logits, tv, ti
    return out


def attn_decode(q, K, V, lens, sinks, window=0):
    """q [B,n_q,D]; K,V [B,S,n_kv,D]; lens [B]; sinks [n_q] -> out [B,n_q,D] (fp32)."""
    q, K, V, sinks, lens = _f32(q), _f32(K), _f32(V), _f32(sinks), _i32(lens)
    B, n_q, D = q.shape
    _, S, n_kv, _ = K.shape
    out = np.empty_like(q)
    lib().orc_attn_decode(_fp(q), _fp(K), _fp(V), _ip(lens), _fp(sinks), C.c_int(B), C.c_int(S),
                          C.c_int(n_q), C.c_int(n_kv), C.c_int(D), C.c_int(window), _fp(out))
    return out


def rope_tables(cfg, n_pos):
    oc = OrcConfig.from_config(cfg)
    half = cfg.head_dim // 2
    cs = np.empty((n_pos, half), np.float32)
    sn = np.empty((n_pos, half), np.float32)
    lib().orc_rope_tables(C.byref(oc), C.c_int(n_pos), _fp(cs), _fp(sn))
    return cs, sn


def mxfp4_dequant(blocks, scales):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    nb = scales.size
    assert blocks.size == nb * 16
    out = np.empty(nb * 32, np.float32)
    lib().orc_mxfp4_dequant(blocks.ctypes.data_as(C.c_void_p), scales.ctypes.data_as(C.c_void_p),
                            C.c_longlong(nb), _fp(out))
    return out.reshape(scales.shape + (32,))


# --------------------------------------------------------------------------- whole model
class Model:
    """One-sequence CPU model over a flat fp32 weight array (the .bin payload)."""

    def __init__(self, cfg, weights_flat, stage=0):
        self.cfg = cfg
        self._w = _f32(weights_flat)
        self._oc = OrcConfig.from_config(cfg)
        assert self._w.size >= lib().orc_weight_floats(C.byref(self._oc))
        self._h = C.c_void_p(lib().orc_model_create(C.byref(self._oc), _fp(self._w),
                                                    C.c_int(stage)))

    def forward(self, token, pos):
        p = lib().orc_forward(self._h, C.c_int(int(token)), C.c_int(int(pos)))
        return np.ctypeslib.as_array(p, shape=(self.cfg.vocab_size,)).copy()

    def x(self):
        p = lib().orc_model_x(self._h)
        return np.ctypeslib.as_array(p, shape=(self.cfg.hidden_dim,)).copy()

    def last_router_gap(self):
        """Smallest gap between the k-th and (k+1)-th router score over the layers of the last
        forward call: how close that call came to picking a different expert."""
        return float(lib().orc_model_last_router_gap(self._h))

    def close(self):
        if self._h and _lib is not None:
            _lib.orc_model_destroy(self._h)
        self._h = None

    def __del__(self):
        self.close()


def generate(cfg, weights_flat, prompts, max_seq_len, stage=0, want_margins=False):
    """Greedy decode with the getp loop semantics.  prompts: int32 [n_req, n_prompt].
    Returns (out [n_req, max_seq_len+1] terminated by -1, n_generated[, margins])."""
    w = _f32(weights_flat)
    prompts = _i32(prompts)
    n_req, stride = prompts.shape
    n_prompt = np.full(n_req, stride, np.int32)
    oc = OrcConfig.from_config(cfg)
    out = np.zeros((n_req, max_seq_len + 1), np.int32)
    margins = np.zeros((n_req, max_seq_len + 1), np.float32)
    gap = C.c_float(0)
    n = lib().orc_generate(C.byref(oc), _fp(w), C.c_int(stage), _ip(prompts), _ip(n_prompt),
                           C.c_int(stride), C.c_int(n_req), C.c_int(max_seq_len), _ip(out),
                           _fp(margins), C.byref(gap))
    generate.last_min_router_gap = float(gap.value)
    if want_margins:
        return out, int(n), margins
    return out, int(n)


def ref_generate(bin_path, prompts, max_seq_len):
    """Same loop, run by the compiled reference CPU model on a .bin file."""
    prompts = _i32(prompts)
    n_req, stride = prompts.shape
    n_prompt = np.full(n_req, stride, np.int32)
    out = np.zeros((n_req, max_seq_len + 1), np.int32)
    n = ref().ref_generate(bin_path.encode(), _ip(prompts), _ip(n_prompt), C.c_int(stride),
                           C.c_int(n_req), C.c_int(max_seq_len), _ip(out))
    return out, int(n)
