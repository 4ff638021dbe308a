"""ctypes front end of oracle/libgd_oracle.so (the CPU checker).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark.  The product package never imports it.

Arrays are numpy; F16 tensors travel as ``np.float16`` (reinterpreted as the
uint16 bit patterns the C side works on).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgd_oracle.so")


def build(force=False):
    """Compile gd_oracle.c with gcc (the Makefile next to this file)."""
    if force or not os.path.exists(_LIB_PATH):
        args = ["make", "-C", _HERE] + (["-B"] if force else [])
        subprocess.run(args, check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_vp, _i64, _i32, _f32, _u64 = C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_uint64


def _declare(l):
    l.gdo_f32_to_f16.restype = C.c_uint16
    l.gdo_f32_to_f16.argtypes = [_f32]
    l.gdo_f16_to_f32.restype = _f32
    l.gdo_f16_to_f32.argtypes = [C.c_uint16]
    l.gdo_splitmix64.restype = _u64
    l.gdo_splitmix64.argtypes = [_u64]
    l.gdo_attn_allowed.restype = C.c_int
    l.gdo_attn_allowed.argtypes = [C.c_int] * 5
    sig = {
        "gdo_f32_to_f16_array": [_vp, _vp, C.c_size_t],
        "gdo_f16_to_f32_array": [_vp, _vp, C.c_size_t],
        "gdo_fill_normal": [_vp, C.c_size_t, _u64, _f32],
        "gdo_fill_normal_f16": [_vp, C.c_size_t, _u64, _f32],
        "gdo_fill_uniform_i32": [_vp, C.c_size_t, _u64, _i32, _i32],
        "gdo_rand_uniform_f32": [_vp, C.c_size_t, _u64, C.c_float, C.c_float],
        "gdo_fill_tokens": [_vp, C.c_uint32, _f32],
        "gdo_fill_values": [_vp, C.c_size_t, _f32, _f32],
        "gdo_kv_cache_append": [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _i64, _i64],
        "gdo_kv_cache_append_packed": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64],
        "gdo_sdpa_decode_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32,
                                C.c_int, C.c_int, _vp],
        "gdo_sdpa_decode_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32,
                                C.c_int, C.c_int, _vp],
        "gdo_sdpa_varlen_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, C.c_int, C.c_int,
                                C.c_int, _i64, _vp],
        "gdo_rms_norm_f16": [_vp, _vp, _i64, _i64, _f32, _vp],
        "gdo_rms_norm_f32": [_vp, _vp, _i64, _i64, _f32, _vp],
        "gdo_qkv_split_rope_f16": [_vp, _vp, _i64, _i64, _i64, _f32, C.c_int, _vp, _vp, _vp],
        "gdo_linear_nt_f16": [_vp, _vp, _vp, _i64, _i64, _i64, _vp],
        "gdo_linear_f16": [_vp, _vp, _vp, _i64, _i64, _i64, _vp],
        "gdo_add_f16": [_vp, _vp, _i64, _i64, _vp],
        "gdo_swiglu_split_f16": [_vp, _i64, _i64, _vp],
        "gdo_embedding_f16": [_vp, _vp, _i64, _i64, _i64, _vp],
        "gdo_argmax_rows_f16": [_vp, _i64, _i64, _vp, _vp],
        "gdo_logits_softcap": [_vp, _i64, _f32],
        "gdo_minimax_m3_index_topk_f16": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
        "gdo_minimax_m3_sparse_attention_f16": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp],
        "gdo_repetition_penalty": [_vp, _i64, _vp, _i64, _f32],
        "gdo_decoder_destroy": [_vp],
        "gdo_decoder_untie_lm_head": [_vp, _u64],
        "gdo_decoder_set_minimax_m3": [_vp, _i64, _i64, _i64, _i64],
        "gdo_decoder_step": [_vp, _vp, _vp, _vp, _vp],
        "gdo_decoder_prefill": [_vp, _vp, _vp, _vp, _vp, _vp, _vp],
    }
    for name, argtypes in sig.items():
        fn = getattr(l, name)
        fn.restype = None
        fn.argtypes = argtypes
    l.gdo_sample_next_token.restype = C.c_int32
    l.gdo_sample_next_token.argtypes = [_vp, _i64, _vp, _i64, _f32, _f32, _f32, C.POINTER(_u64), C.POINTER(C.c_double)]
    l.gdo_decoder_create.restype = _vp
    l.gdo_decoder_create.argtypes = [_i64] * 8 + [C.c_int, _u64]
    l.gdo_decoder_tensor.restype = _vp
    l.gdo_decoder_tensor.argtypes = [_vp, C.c_char_p, _i64]
    l.gdo_decoder_positions.restype = _vp
    l.gdo_decoder_positions.argtypes = [_vp]


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# ---- conversions and generators -------------------------------------------

def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().gdo_f32_to_f16_array(_p(x), _p(out), x.size)
    return out


def f16_bits_to_f32(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().gdo_f16_to_f32_array(_p(bits), _p(out), bits.size)
    return out


def splitmix64(x):
    return int(lib().gdo_splitmix64(x & 0xFFFFFFFFFFFFFFFF))


def fill_normal(count, seed, stddev):
    out = np.empty(count, np.float32)
    lib().gdo_fill_normal(_p(out), count, seed & 0xFFFFFFFFFFFFFFFF, stddev)
    return out


def normal_f16(shape, seed, stddev=1.0):
    n = int(np.prod(shape))
    out = np.empty(n, np.uint16)
    lib().gdo_fill_normal_f16(_p(out), n, seed & 0xFFFFFFFFFFFFFFFF, stddev)
    return out.view(np.float16).reshape(shape)


def rand_uniform_f32(count, seed, low, high):
    out = np.empty(count, np.float32)
    lib().gdo_rand_uniform_f32(_p(out), count, seed & 0xFFFFFFFFFFFFFFFF, low, high)
    return out


def uniform_i32(count, seed, lo, hi):
    out = np.empty(count, np.int32)
    lib().gdo_fill_uniform_i32(_p(out), count, seed & 0xFFFFFFFFFFFFFFFF, lo, hi)
    return out


def fill_tokens(count, base):
    out = np.empty(count, np.uint16)
    lib().gdo_fill_tokens(_p(out), count, base)
    return out.view(np.float16)


def fill_values(count, scale, bias):
    out = np.empty(count, np.float32)
    lib().gdo_fill_values(_p(out), count, scale, bias)
    return out


# ---- operators --------------------------------------------------------------

def kv_cache_append(k_cache, v_cache, k_new, v_new, pos):
    """In place.  caches [B,Tmax,H,D], new [B,Tnew,H,D]; pos int or int32 [B]."""
    B, tmax = k_cache.shape[0], k_cache.shape[1]
    tnew = k_new.shape[1]
    row_bytes = k_cache.shape[2] * k_cache.shape[3] * k_cache.itemsize
    assert all(a.flags.c_contiguous for a in (k_cache, v_cache, k_new, v_new))
    if np.isscalar(pos):
        lib().gdo_kv_cache_append(_p(k_cache), _p(v_cache), _p(k_new), _p(v_new), None, int(pos),
                                  B, tnew, tmax, row_bytes)
    else:
        pos = _c(pos, np.int32)
        lib().gdo_kv_cache_append(_p(k_cache), _p(v_cache), _p(k_new), _p(v_new), _p(pos), 0,
                                  B, tnew, tmax, row_bytes)


def kv_cache_append_packed(k_cache, v_cache, k_new, v_new, pos, cu):
    """In place.  caches [B,Tmax,H,D], new [N,H,D], pos [B], cu [B+1]."""
    B, tmax = k_cache.shape[0], k_cache.shape[1]
    row_bytes = k_cache.shape[2] * k_cache.shape[3] * k_cache.itemsize
    pos, cu = _c(pos, np.int32), _c(cu, np.int32)
    assert all(a.flags.c_contiguous for a in (k_cache, v_cache, k_new, v_new))
    lib().gdo_kv_cache_append_packed(_p(k_cache), _p(v_cache), _p(k_new), _p(v_new), _p(pos),
                                     _p(cu), B, k_new.shape[0], tmax, row_bytes)


def attn_allowed(i, j, causal, window, prefix):
    return bool(lib().gdo_attn_allowed(i, j, int(causal), window, prefix))


def sdpa_decode(q, k, v, pos, scale, window=0, prefix=0, out_init=None):
    """q [B,Tq,Hq,D]; k,v [B,Tmax,Hkv,D]; pos int32 [B].  Returns float32 (unrounded)."""
    B, Tq, Hq, D = q.shape
    Tmax, Hkv = k.shape[1], k.shape[2]
    pos = _c(np.broadcast_to(np.asarray(pos, np.int32), (B,)), np.int32)
    out = np.zeros(q.shape, np.float32) if out_init is None else _c(out_init, np.float32).copy()
    if q.dtype == np.float16:
        q, k, v = (_c(a, np.float16) for a in (q, k, v))
        lib().gdo_sdpa_decode_f16(_p(q), _p(k), _p(v), _p(pos), B, Tq, Tmax, Hq, Hkv, D, scale,
                                  window, prefix, _p(out))
    else:
        q, k, v = (_c(a, np.float32) for a in (q, k, v))
        lib().gdo_sdpa_decode_f32(_p(q), _p(k), _p(v), _p(pos), B, Tq, Tmax, Hq, Hkv, D, scale,
                                  window, prefix, _p(out))
    return out


def sdpa_varlen(q, k, v, cu, scale, causal=True, window=0, prefix=0, max_seqlen=0):
    """q [N,Hq,D]; k,v [N,Hkv,D] float16; cu int32 [B+1].  Returns float32."""
    N, Hq, D = q.shape
    Hkv = k.shape[1]
    cu = _c(cu, np.int32)
    q, k, v = (_c(a, np.float16) for a in (q, k, v))
    out = np.zeros(q.shape, np.float32)
    lib().gdo_sdpa_varlen_f16(_p(q), _p(k), _p(v), _p(cu), len(cu) - 1, Hq, Hkv, D, scale,
                              int(causal), window, prefix, max_seqlen, _p(out))
    return out


def rms_norm(x, w, eps):
    rows, cols = int(np.prod(x.shape[:-1])), x.shape[-1]
    if x.dtype == np.float16:
        x, w = _c(x, np.float16), _c(w, np.float16)
        out = np.empty(x.shape, np.float16)
        lib().gdo_rms_norm_f16(_p(x), _p(w), rows, cols, eps, _p(out))
    else:
        x, w = _c(x, np.float32), _c(w, np.float32)
        out = np.empty(x.shape, np.float32)
        lib().gdo_rms_norm_f32(_p(x), _p(w), rows, cols, eps, _p(out))
    return out


def qkv_split_rope(qkv, pos, n_heads, head_dim, theta=10000.0, interleaved=False):
    qkv, pos = _c(qkv, np.float16), _c(pos, np.int32)
    N = qkv.shape[0]
    q, k, v = (np.empty((N, n_heads, head_dim), np.float16) for _ in range(3))
    lib().gdo_qkv_split_rope_f16(_p(qkv), _p(pos), N, n_heads, head_dim, theta, int(interleaved),
                                 _p(q), _p(k), _p(v))
    return q, k, v


def linear_nt(x, w, bias=None):
    """y = half(half(x @ w.T) + bias); w [N,K]."""
    x, w = _c(x, np.float16), _c(w, np.float16)
    bias = None if bias is None else _c(bias, np.float16)
    M, K, N = int(np.prod(x.shape[:-1])), x.shape[-1], w.shape[0]
    y = np.empty(x.shape[:-1] + (N,), np.float16)
    lib().gdo_linear_nt_f16(_p(x), _p(w), _p(bias), M, K, N, _p(y))
    return y


def linear(x, w, bias=None):
    """y = half(x @ w + bias); w [K,N]."""
    x, w = _c(x, np.float16), _c(w, np.float16)
    bias = None if bias is None else _c(bias, np.float16)
    M, K, N = int(np.prod(x.shape[:-1])), x.shape[-1], w.shape[1]
    y = np.empty(x.shape[:-1] + (N,), np.float16)
    lib().gdo_linear_f16(_p(x), _p(w), _p(bias), M, K, N, _p(y))
    return y


def add(x, y):
    x, y = _c(x, np.float16), _c(y, np.float16)
    out = np.empty(x.shape, np.float16)
    lib().gdo_add_f16(_p(x), _p(y), x.size, y.size, _p(out))
    return out


def swiglu_split(x12):
    x12 = _c(x12, np.float16)
    H = x12.shape[-1] // 2
    rows = int(np.prod(x12.shape[:-1]))
    out = np.empty(x12.shape[:-1] + (H,), np.float16)
    lib().gdo_swiglu_split_f16(_p(x12), rows, H, _p(out))
    return out


def swiglu_split_linear(x12, w, bias=None):
    return linear(swiglu_split(x12), w, bias)


def embedding(table, ids):
    table, ids = _c(table, np.float16), _c(ids, np.int32)
    out = np.empty(ids.shape + (table.shape[1],), np.float16)
    lib().gdo_embedding_f16(_p(table), _p(ids), ids.size, table.shape[0], table.shape[1], _p(out))
    return out


def argmax_rows(logits):
    logits = _c(logits, np.float16)
    rows, cols = logits.shape
    ids = np.empty(rows, np.int32)
    gap = np.empty(rows, np.float32)
    lib().gdo_argmax_rows_f16(_p(logits), rows, cols, _p(ids), _p(gap))
    return ids, gap


def minimax_m3_index_topk(q, k, cu, block, topk, init_blocks=1, local_blocks=1):
    """q, k [N,H,Dh] F16, cu [B+1] -> block ids [H,N,topk]."""
    q, k, cu = _c(q, np.float16), _c(k, np.float16), _c(cu, np.int32)
    N, H, Dh = q.shape
    out = np.empty((H, N, topk), np.int32)
    lib().gdo_minimax_m3_index_topk_f16(_p(q), _p(k), _p(cu), cu.size - 1, H, Dh, block, topk, init_blocks,
                                        local_blocks, _p(out))
    return out


def minimax_m3_sparse_attention(q, k, v, cu, topk_idx, block, scale):
    """q [N,Hq,Dh], k / v [N,Hkv,Dh], topk_idx [Hkv,N,topk] -> out [N,Hq,Dh] F16."""
    q, k, v = _c(q, np.float16), _c(k, np.float16), _c(v, np.float16)
    cu, topk_idx = _c(cu, np.int32), _c(topk_idx, np.int32)
    N, Hq, Dh = q.shape
    out = np.empty((N, Hq, Dh), np.float16)
    lib().gdo_minimax_m3_sparse_attention_f16(_p(q), _p(k), _p(v), _p(cu), _p(topk_idx), cu.size - 1, Hq, k.shape[1],
                                              Dh, block, topk_idx.shape[2], scale, _p(out))
    return out


def logits_softcap(logits, cap):
    out = _c(logits, np.float32).copy()
    lib().gdo_logits_softcap(_p(out), out.size, cap)
    return out


def repetition_penalty(logits, history, penalty):
    out = _c(logits, np.float32).copy()
    history = _c(history, np.int32)
    lib().gdo_repetition_penalty(_p(out), out.size, _p(history), history.size, penalty)
    return out


def sample_next_token(logits, history, temperature, min_p, penalty, rng):
    """One row.  Returns (token, new rng state, margin, logits after the penalty)."""
    work = _c(logits, np.float32).copy()
    history = _c(history, np.int32)
    state, margin = _u64(rng), C.c_double()
    token = lib().gdo_sample_next_token(_p(work), work.size, _p(history), history.size, temperature, min_p, penalty,
                                        C.byref(state), C.byref(margin))
    return int(token), int(state.value), float(margin.value), work


# ---- decoder -------------------------------------------------------------------

class Decoder:
    """CPU decoder following the reference example's call sequence."""

    _SHAPES = {
        "embed": lambda d: (d.vocab, d.d_model), "lm_head": lambda d: (d.vocab, d.d_model), "lm_bias": lambda d: (d.vocab,),
        "final_norm": lambda d: (d.d_model,), "attn_norm": lambda d: (d.d_model,),
        "mlp_norm": lambda d: (d.d_model,), "w_qkv": lambda d: (3 * d.d_model, d.d_model),
        "b_qkv": lambda d: (3 * d.d_model,), "w_attn": lambda d: (d.d_model, d.d_model),
        "b_attn": lambda d: (d.d_model,), "w_upgate": lambda d: (2 * d.mlp_hidden, d.d_model),
        "b_upgate": lambda d: (2 * d.mlp_hidden,), "w_down": lambda d: (d.mlp_hidden, d.d_model),
        "b_down": lambda d: (d.d_model,),
        "k_cache": lambda d: (d.batch, d.max_seq, d.n_heads, d.head_dim),
        "v_cache": lambda d: (d.batch, d.max_seq, d.n_heads, d.head_dim),
    }

    def __init__(self, vocab, d_model, n_layers, n_heads, head_dim, mlp_hidden, max_seq, batch,
                 window=0, seed=1000, tie_lm_head=True):
        self.vocab, self.d_model, self.n_layers = vocab, d_model, n_layers
        self.n_heads, self.head_dim, self.mlp_hidden = n_heads, head_dim, mlp_hidden
        self.max_seq, self.batch, self.window, self.seed = max_seq, batch, window, seed
        self._h = lib().gdo_decoder_create(vocab, d_model, n_layers, n_heads, head_dim, mlp_hidden,
                                           max_seq, batch, window, seed)
        if not tie_lm_head:
            lib().gdo_decoder_untie_lm_head(self._h, seed)

    def set_minimax_m3(self, block, topk, init_blocks=1, local_blocks=1):
        """MiniMax-M3 architecture: the packed prefill attends over picked blocks when the context is long enough."""
        lib().gdo_decoder_set_minimax_m3(self._h, block, topk, init_blocks, local_blocks)

    def close(self):
        if self._h:
            lib().gdo_decoder_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def tensor(self, name, layer=0):
        """numpy float16 view of a weight or cache owned by the C decoder."""
        shape = self._SHAPES[name](self)
        ptr = lib().gdo_decoder_tensor(self._h, name.encode(), layer)
        n = int(np.prod(shape))
        buf = (C.c_uint16 * n).from_address(ptr)
        return np.frombuffer(buf, np.float16).reshape(shape)

    @property
    def positions(self):
        ptr = lib().gdo_decoder_positions(self._h)
        return np.frombuffer((C.c_int32 * self.batch).from_address(ptr), np.int32)

    def step(self, ids):
        ids = _c(ids, np.int32)
        logits = np.empty((self.batch, self.vocab), np.float16)
        nxt = np.empty(self.batch, np.int32)
        gap = np.empty(self.batch, np.float32)
        lib().gdo_decoder_step(self._h, _p(ids), _p(logits), _p(nxt), _p(gap))
        return logits, nxt, gap

    def prefill(self, ids, cu, want_hidden=False):
        ids, cu = _c(ids, np.int32), _c(cu, np.int32)
        logits = np.empty((self.batch, self.vocab), np.float16)
        nxt = np.empty(self.batch, np.int32)
        gap = np.empty(self.batch, np.float32)
        hidden = np.empty((len(ids), self.d_model), np.float16) if want_hidden else None
        lib().gdo_decoder_prefill(self._h, _p(ids), _p(cu), _p(logits), _p(nxt), _p(gap), _p(hidden))
        return (logits, nxt, gap, hidden) if want_hidden else (logits, nxt, gap)
