"""Thin Python front end over the C ABI for tests and benchmarks.

PyTorch is used only to own device memory and streams; every computation below is a call into
``libgptoss_mi355.so`` with raw device pointers.  Function names follow the reference's op layer
(``getp-csrc/include/layer_hip_batch.hpp``, ``kernel.hpp``, ``flash_attn_hip.hpp``)."""
from __future__ import annotations

import ctypes as C

import torch

from . import lib as _l


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("gptoss_mi355 needs a GPU: there is no CPU path")


def pack_weight(w: torch.Tensor, glu: bool = False) -> torch.Tensor:
    """w: [n_mat, n_out, n_in] (or 2-D) bf16/fp32 on the GPU -> packed bf16 tensor (flat)."""
    _need_gpu()
    L = _l.load()
    if w.dim() == 2:
        w = w.unsqueeze(0)
    w = w.contiguous()
    n_mat, n_out, n_in = w.shape
    flags = (_l.PACK_GLU if glu else 0)
    if w.dtype == torch.float32:
        flags |= _l.PACK_SRC_FP32
    elif w.dtype != torch.bfloat16:
        raise TypeError("pack_weight: bf16 or fp32 expected")
    out = torch.empty(n_mat * n_out * n_in, dtype=torch.bfloat16, device=w.device)
    _l.check(L.gptoss_pack_weight(_ptr(w), _ptr(out), n_mat, n_out, n_in, flags, _stream()))
    return out


def router_gemm(t, w_router, b_router):
    _need_gpu()
    L = _l.load()
    B, H = t.shape
    E = w_router.shape[0]
    logits = torch.empty(B, E, dtype=torch.float32, device=t.device)
    _l.check(L.gptoss_router_gemm(_ptr(t), _ptr(w_router), _ptr(b_router), _ptr(logits), B, H, E,
                                  _stream()))
    return logits


def moe_route(logits, k, rows_per_tile=0):
    """-> topk_w [B,k], topk_i [B,k], expert_offsets [E+1], sorted_pair_ids [B*k], inv_perm [B*k],
    tiles (or None)."""
    _need_gpu()
    L = _l.load()
    B, E = logits.shape
    dev = logits.device
    topk_w = torch.empty(B, k, dtype=torch.float32, device=dev)
    topk_i = torch.empty(B, k, dtype=torch.int32, device=dev)
    off = torch.empty(E + 1, dtype=torch.int32, device=dev)
    srt = torch.full((B * k,), -1, dtype=torch.int32, device=dev)
    inv = torch.full((B * k,), -1, dtype=torch.int32, device=dev)
    tiles = None
    if rows_per_tile:
        n = L.gptoss_moe_max_tiles(B, k, E, rows_per_tile)
        tiles = torch.full((1 + 3 * n,), -1, dtype=torch.int32, device=dev)
    _l.check(L.gptoss_moe_route(_ptr(logits), B, E, k, _ptr(topk_w), _ptr(topk_i), _ptr(off),
                                _ptr(srt), _ptr(inv), _ptr(tiles), rows_per_tile, _stream()))
    return topk_w, topk_i, off, srt, inv, tiles


class MoeLayer:
    """Device weights of one MoE block in the layout the kernels read, plus a workspace."""

    def __init__(self, w_router, b_router, w1, b1, w2, b2, top_k=4, swiglu_limit=7.0,
                 max_tokens=1024):
        _need_gpu()
        self.L = _l.load()
        E, H = w_router.shape
        I = w2.shape[2]
        assert tuple(w1.shape) == (E, 2 * I, H) and tuple(w2.shape) == (E, H, I)
        self.E, self.H, self.I, self.k = E, H, I, top_k
        dev = w_router.device
        self.w_router = w_router.to(torch.bfloat16).contiguous()
        self.b_router = b_router.to(torch.float32).contiguous()
        self.w1 = pack_weight(w1, glu=True)
        self.b1 = b1.to(torch.float32).contiguous()
        self.w2 = pack_weight(w2)
        self.b2 = b2.to(torch.float32).contiguous()
        self.desc = _l.MoeWeights(E, top_k, H, I, swiglu_limit, self.w_router.data_ptr(),
                                  self.b_router.data_ptr(), self.w1.data_ptr(),
                                  self.b1.data_ptr(), self.w2.data_ptr(), self.b2.data_ptr())
        self.max_tokens = max_tokens
        self.ws_bytes = self.L.gptoss_moe_workspace_bytes(max_tokens, E, top_k, H, I)
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device=dev)
        self._last_B = 0

    def forward(self, t, out=None, accumulate=False):
        B = t.shape[0]
        assert B <= self.max_tokens and t.dtype == torch.bfloat16 and t.is_contiguous()
        if out is None:
            out = torch.empty(B, self.H, dtype=torch.float32, device=t.device)
        _l.check(self.L.gptoss_moe_forward(C.byref(self.desc), _ptr(t), B, _ptr(out),
                                           1 if accumulate else 0, _ptr(self.ws), self.ws_bytes,
                                           _stream()))
        self._last_B = B
        return out

    def routing_views(self):
        """Routing results of the last forward call as torch tensors (copies)."""
        B, E, k = self._last_B, self.E, self.k
        ptrs = [C.c_void_p() for _ in range(6)]
        _l.check(self.L.gptoss_moe_workspace_views(_ptr(self.ws), B, E, k, self.H, self.I,
                                                   *[C.byref(p) for p in ptrs]))
        base = self.ws.data_ptr()
        shapes = [((B, E), torch.float32), ((B, k), torch.float32), ((B, k), torch.int32),
                  ((E + 1,), torch.int32), ((B * k,), torch.int32), ((B * k,), torch.int32)]
        out = []
        for p, (shape, dt) in zip(ptrs, shapes):
            off = p.value - base
            n = 1
            for s in shape:
                n *= s
            out.append(self.ws[off:off + n * 4].view(dt).view(shape).clone())
        return out


class KVCache:
    """bf16 K/V cache of one layer in the kernels' internal layout."""

    def __init__(self, B, n_kv, head_dim, capacity, device="cuda", zero=False):
        _need_gpu()
        self.L = _l.load()
        self.B, self.n_kv, self.D, self.cap = B, n_kv, head_dim, capacity
        nbytes = self.L.gptoss_kv_cache_bytes(B, n_kv, head_dim, capacity)
        if nbytes == 0 or capacity % 64:
            raise ValueError("KVCache: capacity must be a positive multiple of 64")
        alloc = torch.zeros if zero else torch.empty
        #: K and V together, in the kernels' block layout
        self.kv = alloc(nbytes // 2, dtype=torch.bfloat16, device=device)

    def write(self, k_rows, v_rows, pos0=0):
        """k_rows, v_rows: bf16 [B, n_tok, n_kv, D] for positions pos0 .. pos0+n_tok-1."""
        B, n_tok, n_kv, D = k_rows.shape
        assert (B, n_kv, D) == (self.B, self.n_kv, self.D)
        assert k_rows.dtype == torch.bfloat16 and v_rows.dtype == torch.bfloat16
        k_rows, v_rows = k_rows.contiguous(), v_rows.contiguous()
        _l.check(self.L.gptoss_kv_cache_write(_ptr(self.kv), _ptr(k_rows), _ptr(v_rows), B, n_kv, D,
                                              self.cap, pos0, n_tok, _stream()))

    def first(self, n_seq):
        """A view of the first n_seq sequences (the layout is sequence-major)."""
        c = KVCache.__new__(KVCache)
        c.L, c.B, c.n_kv, c.D, c.cap = self.L, n_seq, self.n_kv, self.D, self.cap
        c.kv = self.kv[: self.L.gptoss_kv_cache_bytes(n_seq, self.n_kv, self.D, self.cap) // 2]
        return c


class AttnDecode:
    """single_query_attn_flash_batched: q [B,n_q,D] fp32 -> out [B,n_q,D] bf16."""

    def __init__(self, B, n_q, n_kv, head_dim, max_len, device="cuda"):
        _need_gpu()
        self.L = _l.load()
        self.B, self.n_q, self.n_kv, self.D, self.max_len = B, n_q, n_kv, head_dim, max_len
        self.ws_bytes = self.L.gptoss_attn_workspace_bytes(B, n_q, n_kv, head_dim, max_len)
        self.ws = torch.empty(max(self.ws_bytes, 256), dtype=torch.uint8, device=device)

    def forward(self, q, cache: KVCache, lens, sinks=None, window=0, out=None, max_len=None):
        B = q.shape[0]
        assert q.dtype == torch.float32 and q.is_contiguous() and (lens is None or lens.dtype == torch.int32)
        if out is None:
            out = torch.empty(B, self.n_q, self.D, dtype=torch.bfloat16, device=q.device)
        _l.check(self.L.gptoss_attn_decode(_ptr(q), _ptr(cache.kv), _ptr(lens),
                                           _ptr(sinks), _ptr(out), B, self.n_q, self.n_kv, self.D,
                                           cache.cap, window, max_len or self.max_len,
                                           _ptr(self.ws), self.ws_bytes, _stream()))
        return out


def attn_decode_static(q, cache: KVCache, lens, n_q, sinks=None, window=0, max_len=None, out=None):
    """gptoss_attn_decode_static: the decode attention on the library's built-in scratch (no workspace,
    no allocation inside the call; `out` is the caller's)."""
    _need_gpu()
    L = _l.load()
    B = q.shape[0]
    assert q.dtype == torch.float32 and q.is_contiguous() and lens.dtype == torch.int32
    if out is None:
        out = torch.empty(B, n_q, cache.D, dtype=torch.bfloat16, device=q.device)
    _l.check(L.gptoss_attn_decode_static(_ptr(q), _ptr(cache.kv), _ptr(lens), _ptr(sinks),
                                         _ptr(out), B, n_q, cache.n_kv, cache.D, cache.cap, window,
                                         int(max_len), _stream()))
    return out


class AttnPrefill:
    """The decode attention for T consecutive positions of every sequence at once:
    q [B,T,n_q,D] fp32 -> out [B,T,n_q,D] bf16; row (b,t) sees cached positions <= pos0 + t."""

    def __init__(self, B, T, n_q, n_kv, head_dim, max_len, device="cuda"):
        _need_gpu()
        self.L = _l.load()
        self.n_q, self.n_kv, self.D = n_q, n_kv, head_dim
        self.ws_bytes = self.L.gptoss_attn_prefill_workspace_bytes(B, T, n_q, n_kv, head_dim, max_len)
        self.ws = torch.empty(max(self.ws_bytes, 256), dtype=torch.uint8, device=device)

    def forward(self, q, cache: KVCache, pos0=0, sinks=None, window=0):
        B, T = q.shape[:2]
        assert q.dtype == torch.float32 and q.is_contiguous()
        out = torch.empty(B, T, self.n_q, self.D, dtype=torch.bfloat16, device=q.device)
        _l.check(self.L.gptoss_attn_prefill(_ptr(q), _ptr(cache.kv), _ptr(sinks), _ptr(out),
                                            B, T, pos0, self.n_q, self.n_kv, self.D, cache.cap, window,
                                            _ptr(self.ws), self.ws_bytes, _stream()))
        return out


# ---- glue ops (names follow getp-csrc/include/layer_hip_batch.hpp) -------------------------------
def embedding_lookup(table, tokens):
    """table bf16 [V,H], tokens int32 [B] -> fp32 [B,H]."""
    _need_gpu()
    V, H = table.shape
    x = torch.empty(tokens.numel(), H, dtype=torch.float32, device=table.device)
    _l.check(_l.load().gptoss_embedding(_ptr(table), _ptr(tokens), _ptr(x), tokens.numel(), H, V, _stream()))
    return x


def rmsnorm(x, weight, residual=None):
    """x fp32 [B,H] (updated in place by += residual when given) -> bf16 [B,H]."""
    _need_gpu()
    B, H = x.shape
    t = torch.empty(B, H, dtype=torch.bfloat16, device=x.device)
    _l.check(_l.load().gptoss_rmsnorm(_ptr(x), _ptr(residual), _ptr(weight), _ptr(t), B, H, _stream()))
    return t


def dense_gemm(a, w_packed, n_out, bias=None, out=None):
    """a bf16 [B,K], w_packed = pack_weight(w [n_out,K]) -> fp32 [B,n_out]."""
    _need_gpu()
    B, K = a.shape
    if out is None:
        out = torch.empty(B, n_out, dtype=torch.float32, device=a.device)
    _l.check(_l.load().gptoss_dense_gemm(_ptr(a), _ptr(w_packed), _ptr(bias), _ptr(out), B, n_out, K, _stream()))
    return out


def classifier_argmax(a, w_packed, vocab):
    """arg max over the vocabulary of a . w^T without the logits: a bf16 [B,K] -> int32 [B]."""
    _need_gpu()
    L = _l.load()
    B, K = a.shape
    nb = L.gptoss_classifier_argmax_workspace_bytes(B, vocab)
    ws = torch.empty(max(nb, 256), dtype=torch.uint8, device=a.device)
    ids = torch.empty(B, dtype=torch.int32, device=a.device)
    _l.check(L.gptoss_classifier_argmax(_ptr(a), _ptr(w_packed), _ptr(ids), B, vocab, K, _ptr(ws), nb, _stream()))
    return ids


def argmax(logits):
    _need_gpu()
    B, V = logits.shape
    ids = torch.empty(B, dtype=torch.int32, device=logits.device)
    _l.check(_l.load().gptoss_argmax(_ptr(logits), _ptr(ids), B, V, _stream()))
    return ids


def rope_tables(cfg, n_pos):
    """-> (cos, sin) float32 numpy arrays [n_pos, head_dim/2] (host)."""
    import numpy as np
    cc = _l.Config.from_config(cfg)
    cs = np.empty((n_pos, cfg.head_dim // 2), np.float32)
    sn = np.empty_like(cs)
    _l.check(_l.load().gptoss_rope_tables(C.byref(cc), n_pos, cs.ctypes.data_as(C.c_void_p),
                                          sn.ctypes.data_as(C.c_void_p)))
    return cs, sn


def rope_kv_store(qkv, cache: KVCache, cos_t, sin_t, lens, n_q):
    """qkv fp32 [B,(n_q+2n_kv)*D]; rotates q and k for position lens[b]-1, stores k, v into the cache;
    -> q fp32 [B,n_q,D]."""
    _need_gpu()
    B = qkv.shape[0]
    q = torch.empty(B, n_q, cache.D, dtype=torch.float32, device=qkv.device)
    _l.check(_l.load().gptoss_rope_kv_store(_ptr(qkv), _ptr(q), _ptr(cache.kv), _ptr(cos_t), _ptr(sin_t),
                                            _ptr(lens), B, n_q, cache.n_kv, cache.D, cache.cap, _stream()))
    return q


class KernelTrace:
    """Per-kernel HIP-event timing of the entry points called inside the ``with`` block
    (events are recorded on the stream each kernel is launched on)."""

    def __init__(self, capacity=4096):
        _need_gpu()
        self.L = _l.load()
        self.capacity = capacity
        self._start = [torch.cuda.Event(enable_timing=True) for _ in range(capacity)]
        self._stop = [torch.cuda.Event(enable_timing=True) for _ in range(capacity)]
        # torch creates the underlying hipEvent_t lazily, at the first record()
        for e in self._start + self._stop:
            e.record()
        torch.cuda.synchronize()
        self._sa = (C.c_void_p * capacity)(*[e.cuda_event for e in self._start])
        self._so = (C.c_void_p * capacity)(*[e.cuda_event for e in self._stop])
        self.count = 0

    def __enter__(self):
        _l.check(self.L.gptoss_trace_set(self._sa, self._so, self.capacity))
        return self

    def __exit__(self, *exc):
        # labels are read before the trace is disarmed
        self.count = self.L.gptoss_trace_count()
        self._names = [self.L.gptoss_trace_name(i).decode() for i in range(self.count)]
        self.L.gptoss_trace_set(None, None, 0)
        return False

    def results(self):
        """-> list of (kernel label, milliseconds), in launch order.  Synchronises."""
        torch.cuda.synchronize()
        return [(self._names[i], self._start[i].elapsed_time(self._stop[i]))
                for i in range(self.count)]

    def summary(self):
        """-> {label: (calls, mean ms)}"""
        agg = {}
        for name, ms in self.results():
            c, t = agg.get(name, (0, 0.0))
            agg[name] = (c + 1, t + ms)
        return {k: (c, t / c) for k, (c, t) in agg.items()}


class Engine:
    """Single-GPU decode engine over a flat ``.bin`` payload (or synthetic on-device weights)."""

    def __init__(self, cfg, weights_flat=None, max_batch=8, max_seq=64, synthetic=False,
                 precise=False, seed=0, keep_logits=True, prefill=True, mxfp4_experts=False):
        _need_gpu()
        import numpy as np
        self.L = _l.load()
        self.cfg = cfg
        self.max_batch, self.max_seq = max_batch, max_seq
        flags = (_l.ENGINE_SYNTHETIC if synthetic else 0) | (_l.ENGINE_PRECISE if precise else 0) | \
            (_l.ENGINE_LOGITS if keep_logits else 0) | (0 if prefill else _l.ENGINE_NO_PREFILL) | \
            (_l.ENGINE_MXFP4_EXPERTS if mxfp4_experts else 0)
        self._cc = _l.Config.from_config(cfg)
        wp = None
        if not synthetic:
            self._w = np.ascontiguousarray(weights_flat, dtype=np.float32)
            wp = self._w.ctypes.data_as(C.c_void_p)
        h = C.c_void_p()
        _l.check(self.L.gptoss_engine_create(C.byref(self._cc), wp, max_batch, max_seq, flags,
                                             C.c_uint64(seed), C.byref(h)))
        self._h = h

    def step(self, tokens, pos):
        import numpy as np
        tok = np.ascontiguousarray(tokens, dtype=np.int32)
        nxt = np.empty_like(tok)
        _l.check(self.L.gptoss_engine_step(self._h, tok.ctypes.data_as(C.c_void_p), int(pos),
                                           tok.size, nxt.ctypes.data_as(C.c_void_p)))
        return nxt

    def prefill(self, tokens):
        """Positions 0..T-1 of every sequence (tokens int32 [B, T]) in one pass -> next ids [B]."""
        import numpy as np
        tok = np.ascontiguousarray(tokens, dtype=np.int32)
        B, T = tok.shape
        nxt = np.empty(B, np.int32)
        _l.check(self.L.gptoss_engine_prefill(self._h, tok.ctypes.data_as(C.c_void_p), B, T,
                                              nxt.ctypes.data_as(C.c_void_p)))
        return nxt

    def step_ragged(self, tokens, positions):
        """One step with every sequence at its own position."""
        import numpy as np
        tok = np.ascontiguousarray(tokens, dtype=np.int32)
        pos = np.ascontiguousarray(positions, dtype=np.int32)
        nxt = np.empty_like(tok)
        _l.check(self.L.gptoss_engine_step_ragged(self._h, tok.ctypes.data_as(C.c_void_p),
                                                  pos.ctypes.data_as(C.c_void_p), tok.size,
                                                  nxt.ctypes.data_as(C.c_void_p)))
        return nxt

    def step_rows(self, tokens, slots, positions, sample):
        """One step over arbitrary rows (token, cache slot, position); -> next ids after the rows `sample`."""
        import numpy as np
        tok = np.ascontiguousarray(tokens, dtype=np.int32)
        slot = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(positions, dtype=np.int32)
        smp = np.ascontiguousarray(sample, dtype=np.int32)
        nxt = np.empty(smp.size, np.int32)
        p = lambda a: a.ctypes.data_as(C.c_void_p)
        _l.check(self.L.gptoss_engine_step_rows(self._h, tok.size, p(tok), p(slot), p(pos), smp.size, p(smp), p(nxt)))
        return nxt

    def generate(self, prompts, max_seq_len, n_prompt=None, max_len=None):
        """Greedy generation; max_len (optional, per request) limits a request's total length."""
        import numpy as np
        prompts = np.ascontiguousarray(prompts, dtype=np.int32)
        n_req, stride = prompts.shape
        npr = np.full(n_req, stride, np.int32) if n_prompt is None else \
            np.ascontiguousarray(n_prompt, dtype=np.int32)
        out = np.zeros((n_req, max_seq_len + 1), np.int32)
        n = C.c_longlong(0)
        if max_len is None:
            _l.check(self.L.gptoss_engine_generate(self._h, prompts.ctypes.data_as(C.c_void_p),
                                                   npr.ctypes.data_as(C.c_void_p), stride, n_req,
                                                   max_seq_len, out.ctypes.data_as(C.c_void_p),
                                                   C.byref(n)))
        else:
            ml = np.ascontiguousarray(max_len, dtype=np.int32)
            _l.check(self.L.gptoss_engine_generate_ragged(self._h, prompts.ctypes.data_as(C.c_void_p),
                                                          npr.ctypes.data_as(C.c_void_p), stride, n_req,
                                                          max_seq_len, ml.ctypes.data_as(C.c_void_p),
                                                          out.ctypes.data_as(C.c_void_p), C.byref(n)))
        return out, int(n.value)

    def last_logits(self, B):
        """fp32 [B, vocab] logits of the last step (copied to the host)."""
        lp, xp, nb = C.c_void_p(), C.c_void_p(), C.c_size_t()
        _l.check(self.L.gptoss_engine_debug_views(self._h, C.byref(lp), C.byref(xp), C.byref(nb)))
        if not lp.value:
            raise RuntimeError("the engine was created without keep_logits")
        V = self.cfg.vocab_size
        host = torch.empty(B, V, dtype=torch.float32)
        torch.cuda.synchronize()
        # a plain device-to-host copy of memory the engine owns
        rt = C.CDLL("libamdhip64.so")
        rc = rt.hipMemcpy(C.c_void_p(host.data_ptr()), lp, C.c_size_t(B * V * 4), 2)
        if rc != 0:
            raise RuntimeError(f"hipMemcpy failed: {rc}")
        return host.numpy()

    def tensor(self, name, layer=0):
        """Copy of one weight tensor as the engine holds it on the device (uint8, flat);
        `name` is the tensor's name in binfmt.tensor_shapes."""
        p, n = C.c_void_p(), C.c_size_t()
        _l.check(self.L.gptoss_engine_tensor_view(self._h, _l.TENSORS.index(name), int(layer),
                                                  C.byref(p), C.byref(n)))
        out = torch.empty(n.value, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        rc = C.CDLL("libamdhip64.so").hipMemcpy(C.c_void_p(out.data_ptr()), p, C.c_size_t(n.value), 3)
        if rc != 0:
            raise RuntimeError(f"hipMemcpy failed: {rc}")
        return out

    def device_bytes(self):
        nb = C.c_size_t()
        _l.check(self.L.gptoss_engine_debug_views(self._h, None, None, C.byref(nb)))
        return nb.value

    def close(self):
        if getattr(self, "_h", None):
            self.L.gptoss_engine_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()


def pack_mxfp4(blocks: torch.Tensor, scales: torch.Tensor, glu: bool = False) -> torch.Tensor:
    """blocks uint8 [n_mat, n_out, n_in/2], scales uint8 [n_mat, n_out, n_in/32] -> packed bytes."""
    _need_gpu()
    L = _l.load()
    blocks, scales = blocks.contiguous(), scales.contiguous()
    n_mat, n_out, half = blocks.shape
    n_in = half * 2
    assert tuple(scales.shape) == (n_mat, n_out, n_in // 32)
    out = torch.empty(L.gptoss_packed_mxfp4_bytes(n_mat, n_out, n_in), dtype=torch.uint8,
                      device=blocks.device)
    _l.check(L.gptoss_pack_mxfp4(_ptr(blocks), _ptr(scales), _ptr(out), n_mat, n_out, n_in,
                                 _l.PACK_GLU if glu else 0, _stream()))
    return out


class MoeLayerMxfp4(MoeLayer):
    """MoE block whose expert matrices are MXFP4 (e2m1 codes + one e8m0 scale per 32 inputs)."""

    def __init__(self, w_router, b_router, w1_blocks, w1_scales, b1, w2_blocks, w2_scales, b2,
                 top_k=4, swiglu_limit=7.0, max_tokens=1024):
        _need_gpu()
        self.L = _l.load()
        E, H = w_router.shape
        I = w2_blocks.shape[2] * 2
        assert tuple(w1_blocks.shape) == (E, 2 * I, H // 2) and tuple(w2_blocks.shape) == (E, H, I // 2)
        self.E, self.H, self.I, self.k = E, H, I, top_k
        dev = w_router.device
        self.w_router = w_router.to(torch.bfloat16).contiguous()
        self.b_router = b_router.to(torch.float32).contiguous()
        self.w1 = pack_mxfp4(w1_blocks, w1_scales, glu=True)
        self.b1 = b1.to(torch.float32).contiguous()
        self.w2 = pack_mxfp4(w2_blocks, w2_scales)
        self.b2 = b2.to(torch.float32).contiguous()
        self.desc = _l.MoeWeights(E, top_k, H, I, swiglu_limit, self.w_router.data_ptr(),
                                  self.b_router.data_ptr(), self.w1.data_ptr(),
                                  self.b1.data_ptr(), self.w2.data_ptr(), self.b2.data_ptr())
        self.max_tokens = max_tokens
        self.ws_bytes = self.L.gptoss_moe_workspace_bytes(max_tokens, E, top_k, H, I)
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device=dev)
        self._last_B = 0

    def forward(self, t, out=None, accumulate=False):
        B = t.shape[0]
        assert B <= self.max_tokens and t.dtype == torch.bfloat16 and t.is_contiguous()
        if out is None:
            out = torch.empty(B, self.H, dtype=torch.float32, device=t.device)
        _l.check(self.L.gptoss_moe_forward_mxfp4(C.byref(self.desc), _ptr(t), B, _ptr(out),
                                                 1 if accumulate else 0, _ptr(self.ws),
                                                 self.ws_bytes, _stream()))
        self._last_B = B
        return out
