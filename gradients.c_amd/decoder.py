"""ctypes binding of the host core (gradients_infer.h) and the decoder (gd_gpt_decoder.h)."""
import ctypes as C
import os

import numpy as np

from . import GD_OK, GdError, STATUS_NAMES, lib as _base_lib

_vp = C.c_void_p


class MemoryConfig(C.Structure):  # gd_memory_config
    _fields_ = [("params_bytes", C.c_size_t), ("state_bytes", C.c_size_t), ("scratch_slot_bytes", C.c_size_t),
                ("data_slot_bytes", C.c_size_t), ("scratch_slots", C.c_uint32), ("data_slots", C.c_uint32),
                ("default_alignment", C.c_size_t)]


class GptConfig(C.Structure):  # gd_gpt_config
    _fields_ = [("vocab", C.c_int32), ("d_model", C.c_int32), ("n_layers", C.c_int32), ("n_heads", C.c_int32),
                ("head_dim", C.c_int32), ("mlp_hidden", C.c_int32), ("max_seq", C.c_int32), ("batch", C.c_int32),
                ("sdpa_window", C.c_int32), ("tie_lm_head", C.c_int32), ("rms_eps", C.c_float),
                ("rope_theta", C.c_float), ("seed", C.c_uint64), ("m3_block_size", C.c_int32),
                ("m3_topk_blocks", C.c_int32), ("m3_init_blocks", C.c_int32), ("m3_local_blocks", C.c_int32)]


class Span(C.Structure):  # gd_span
    _fields_ = [("arena", C.c_int), ("slot", C.c_int32), ("offset", C.c_size_t), ("nbytes", C.c_size_t),
                ("alignment", C.c_size_t), ("generation", C.c_uint64), ("buffer", _vp), ("host_ptr", _vp)]


class GdTensor(C.Structure):  # gd_tensor
    _fields_ = [("id", C.c_uint64), ("version", C.c_uint32), ("dtype", C.c_int), ("device", C.c_int),
                ("layout", C.c_int), ("rank", C.c_uint32), ("shape", C.c_int64 * 8), ("strides", C.c_int64 * 8),
                ("storage", Span), ("view_offset", C.c_size_t), ("is_view", C.c_bool), ("requires_grad", C.c_bool),
                ("is_leaf", C.c_bool)]


class Shape(C.Structure):  # gd_shape
    _fields_ = [("rank", C.c_uint32), ("dims", C.c_int64 * 8)]


def make_shape(dims):
    s = Shape()
    s.rank = len(dims)
    for i, d in enumerate(dims):
        s.dims[i] = d
    return s


_T = C.POINTER(GdTensor)


class GptSampling(C.Structure):  # gd_gpt_sampling
    _fields_ = [("temperature", C.c_float), ("min_p", C.c_float), ("repetition_penalty", C.c_float),
                ("logits_softcap", C.c_float), ("stop_token", C.c_int32), ("rng_state", C.c_uint64)]


class CheckpointEntry(C.Structure):  # gd_checkpoint_entry
    _fields_ = [("path", C.c_char * 256), ("flags", C.c_uint32), ("dtype", C.c_int), ("rank", C.c_uint32),
                ("shape", C.c_int64 * 8), ("data_offset", C.c_uint64), ("nbytes", C.c_uint64)]
_declared = False


def lib():
    global _declared
    l = _base_lib()
    if not _declared:
        l.gd_gpt_params_bytes.restype = C.c_size_t
        l.gd_gpt_params_bytes.argtypes = [C.POINTER(GptConfig)]
        l.gd_gpt_state_bytes.restype = C.c_size_t
        l.gd_gpt_state_bytes.argtypes = [C.POINTER(GptConfig)]
        l.gd_gpt_scratch_bytes.restype = C.c_size_t
        l.gd_gpt_scratch_bytes.argtypes = [C.POINTER(GptConfig), C.c_int32]
        l.gd_context_create.argtypes = [C.POINTER(MemoryConfig), C.POINTER(_vp)]
        l.gd_context_destroy.argtypes = [_vp]
        l.gd_context_destroy.restype = None
        l.gd_context_error.argtypes = [_vp]
        l.gd_context_error.restype = C.c_char_p
        l.gd_context_status.argtypes = [_vp]
        l.gd_context_clear_error.argtypes = [_vp]
        l.gd_context_clear_error.restype = None
        l.gd_context_backend.argtypes = [_vp]
        l.gd_context_backend.restype = _vp
        l.gd_context_seal_params.argtypes = [_vp]
        l.gd_batch_empty.restype = _vp
        l.gd_begin_step.argtypes = [_vp, C.c_int, _vp]
        l.gd_end_step.argtypes = [_vp]
        l.gd_synchronize.argtypes = [_vp]
        l.gd_debug_heap_alloc_count.restype = C.c_uint64
        l.gd_debug_set_heap_guard.argtypes = [C.c_bool]
        l.gd_debug_set_heap_guard.restype = None
        l.gd_debug_current_ring_slot.argtypes = [_vp, C.c_int]
        l.gd_debug_ring_slot_generation.argtypes = [_vp, C.c_int, C.c_uint32]
        l.gd_debug_ring_slot_generation.restype = C.c_uint64
        for name in ("gd_alloc_params", "gd_alloc_state", "gd_alloc_scratch", "gd_alloc_data"):
            getattr(l, name).argtypes = [_vp, C.c_size_t, C.c_size_t, C.POINTER(Span)]
        for name in ("gd_tensor_empty", "gd_tensor_zeros", "gd_tensor_ones"):
            getattr(l, name).argtypes = [_vp, C.c_int, C.c_int, Shape, C.c_size_t, _T]
        l.gd_tensor_slice.argtypes = [_vp, _T, C.c_uint32, C.c_int64, C.c_int64, _T]
        l.gd_tensor_validate.argtypes = [_vp, _T]
        l.gd_tensor_is_contiguous.argtypes = [_T]
        l.gd_tensor_is_contiguous.restype = C.c_bool
        l.gd_tensor_write.argtypes = [_vp, _T, _vp, C.c_size_t]
        l.gd_tensor_read.argtypes = [_vp, _T, _vp, C.c_size_t]
        l.gd_tensor_write_f32.argtypes = [_vp, _T, _vp, C.c_size_t]
        l.gd_tensor_read_f32.argtypes = [_vp, _T, _vp, C.c_size_t]
        l.gd_reshape.argtypes = [_vp, _T, Shape, _T]
        l.gd_linear.argtypes = [_vp, _T, _T, _T, _T]
        l.gd_linear_transposed_weight.argtypes = [_vp, _T, _T, _T, _T]
        l.gd_swiglu_split.argtypes = [_vp, _T, _T]
        l.gd_swiglu_split_linear.argtypes = [_vp, _T, _T, _T, _T]
        l.gd_embedding.argtypes = [_vp, _T, _T, _T]
        l.gd_rms_norm.argtypes = [_vp, _T, _T, C.c_float, _T]
        l.gd_add.argtypes = [_vp, _T, _T, _T]
        l.gd_argmax_rows.argtypes = [_vp, _T, _T, _T]
        l.gd_gather_rows.argtypes = [_vp, _T, _T, _T]
        l.gd_kv_cache_append_at.argtypes = [_vp, _T, _T, C.c_int32, _T, _T]
        l.gd_kv_cache_append_positions.argtypes = [_vp, _T, _T, _T, _T, _T]
        l.gd_kv_cache_append_packed.argtypes = [_vp, _T, _T, _T, _T, _T, _T]
        l.gd_sdpa_decode.argtypes = [_vp, _T, _T, _T, _T, _vp, _T]
        l.gd_sdpa_decode_at.argtypes = [_vp, _T, _T, _T, C.c_int32, _vp, _T]
        l.gd_sdpa_decode_positions.argtypes = [_vp, _T, _T, _T, _T, _vp, _T]
        l.gd_sdpa_varlen.argtypes = [_vp, _T, _T, _T, _T, _vp, _T]
        l.gd_qkv_split_rope.argtypes = [_vp, _T, _T, C.c_int32, C.c_int32, _vp, _T, _T, _T]
        l.gd_gpt_decoder_create.argtypes = [_vp, C.POINTER(GptConfig), C.POINTER(_vp)]
        l.gd_gpt_decoder_destroy.argtypes = [_vp]
        l.gd_gpt_decoder_destroy.restype = None
        l.gd_gpt_decoder_tensor.argtypes = [_vp, C.c_char_p, C.c_int32]
        l.gd_gpt_decoder_tensor.restype = _T
        l.gd_gpt_decoder_positions.argtypes = [_vp]
        l.gd_gpt_decoder_positions.restype = C.POINTER(C.c_int32)
        l.gd_gpt_decoder_prefill.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp]
        l.gd_gpt_decoder_step.argtypes = [_vp, _vp, _vp, _vp, _vp]
        l.gd_gpt_decoder_run_resident.argtypes = [_vp, _vp, C.c_int32, _vp, _vp, C.POINTER(C.c_float)]
        l.gd_gpt_decoder_resident_begin.argtypes = [_vp, _vp, C.c_int32, C.c_int32]
        l.gd_gpt_decoder_resident_run.argtypes = [_vp, C.c_int32]
        l.gd_gpt_decoder_resident_sync.argtypes = [_vp]
        l.gd_gpt_decoder_resident_end.argtypes = [_vp, _vp, _vp, C.POINTER(C.c_int32)]
        l.gd_gpt_decoder_load_checkpoint.argtypes = [_vp, C.c_char_p, C.c_int32]
        l.gd_gpt_decoder_generate.argtypes = [_vp, _vp, _vp, C.c_int32, C.POINTER(GptSampling), _vp, _vp]
        l.gd_gpt_decoder_resident_begin_sampled.argtypes = [_vp, _vp, _vp, C.c_int32, C.c_int32, C.POINTER(GptSampling)]
        l.gd_gpt_generation_rng.argtypes = [C.c_uint64, C.c_int32, C.c_uint64]
        l.gd_gpt_generation_rng.restype = C.c_uint64
        l.gd_gpt_config_from_checkpoint.argtypes = [C.c_char_p, C.POINTER(GptConfig)]
        l.gd_checkpoint_read_metadata.argtypes = [C.c_char_p, C.POINTER(_vp), C.POINTER(C.c_size_t)]
        l.gd_checkpoint_open.argtypes = [C.c_char_p, C.POINTER(_vp)]
        l.gd_checkpoint_close.argtypes = [_vp]
        l.gd_checkpoint_close.restype = None
        l.gd_checkpoint_count.argtypes = [_vp]
        l.gd_checkpoint_count.restype = C.c_uint32
        l.gd_checkpoint_entry_at.argtypes = [_vp, C.c_uint32]
        l.gd_checkpoint_entry_at.restype = C.POINTER(CheckpointEntry)
        l.gd_checkpoint_find.argtypes = [_vp, C.c_char_p]
        l.gd_checkpoint_find.restype = C.POINTER(CheckpointEntry)
        l.gd_checkpoint_read.argtypes = [_vp, C.POINTER(CheckpointEntry), C.c_uint64, _vp, C.c_size_t]
        _declared = True
    return l


GD_ARENA_PARAMS, GD_ARENA_STATE, GD_ARENA_SCRATCH, GD_ARENA_DATA = 0, 1, 2, 3
GD_SCOPE_TRAIN, GD_SCOPE_EVAL, GD_SCOPE_INFER = 1, 2, 3


class Context:
    """gd_context: backend + params/state arenas + scratch/data rings."""

    def __init__(self, params_bytes, state_bytes, scratch_slot_bytes, data_slot_bytes=1 << 20, scratch_slots=2,
                 data_slots=2):
        cfg = MemoryConfig(params_bytes, state_bytes, scratch_slot_bytes, data_slot_bytes, scratch_slots, data_slots, 256)
        h = _vp()
        st = lib().gd_context_create(C.byref(cfg), C.byref(h))
        if st != GD_OK:
            raise GdError(st, "gd_context_create (no HIP device? there is no CPU fallback)")
        self.handle = h.value

    def close(self):
        if self.handle:
            lib().gd_context_destroy(self.handle)
            self.handle = None

    def backend(self):
        """Borrowed Backend wrapper around gd_context_backend (for timers and raw operator calls)."""
        from . import Backend
        return Backend(lib().gd_context_backend(self.handle))

    def check(self, st, what):
        if st != GD_OK:
            msg = lib().gd_context_error(self.handle).decode()
            raise GdError(st, f"{what} [{msg}]")

    def error(self):
        return lib().gd_context_error(self.handle).decode()

    def begin_step(self, mode=GD_SCOPE_INFER):
        return lib().gd_begin_step(self.handle, mode, lib().gd_batch_empty())

    def end_step(self):
        return lib().gd_end_step(self.handle)

    def empty(self, arena, dtype, dims, zeros=False):
        t = GdTensor()
        fn = lib().gd_tensor_zeros if zeros else lib().gd_tensor_empty
        st = fn(self.handle, arena, dtype, make_shape(dims), 256, C.byref(t))
        return st, t

    def write(self, t, array):
        a = np.ascontiguousarray(array)
        return lib().gd_tensor_write(self.handle, C.byref(t), a.ctypes.data_as(_vp), a.nbytes)

    def read(self, t, np_dtype):
        shape = tuple(t.shape[i] for i in range(t.rank))
        out = np.empty(shape, np_dtype)
        st = lib().gd_tensor_read(self.handle, C.byref(t), out.ctypes.data_as(_vp), out.nbytes)
        return st, out


def gpt_config(vocab, d_model, n_layers, n_heads, head_dim, mlp_hidden, max_seq, batch, window=0, tie_lm_head=True,
               seed=1000, minimax_m3=None):
    """minimax_m3: (block_size, topk_blocks, init_blocks, local_blocks) for the MiniMax-M3 architecture."""
    m3 = tuple(minimax_m3) if minimax_m3 else (0, 0, 0, 0)
    return GptConfig(vocab, d_model, n_layers, n_heads, head_dim, mlp_hidden, max_seq, batch, window,
                     int(tie_lm_head), 1e-5, 10000.0, seed, *m3)


def config_from_checkpoint(path, batch, max_seq=0, n_heads=0, head_dim=0, window=0, seed=1000):
    """gd_gpt_config for the model stored in a .gdckpt file; the keyword values are used where the file is silent."""
    cfg = GptConfig(0, 0, 0, n_heads, head_dim, 0, max_seq, batch, window, 1, 1e-5, 10000.0, seed)
    st = lib().gd_gpt_config_from_checkpoint(os.fsencode(path), C.byref(cfg))
    if st != GD_OK:
        raise GdError(st, f"gd_gpt_config_from_checkpoint({path})")
    return cfg


class GptDecoder:
    """The decoder of gd_gpt_decoder.h with its own context sized for the configuration."""

    def __init__(self, cfg, scratch_slot_bytes=None, max_prefill_tokens=0):
        self.cfg = cfg
        l = lib()
        rows = max(cfg.batch, max_prefill_tokens)
        if scratch_slot_bytes is None:
            scratch_slot_bytes = l.gd_gpt_scratch_bytes(C.byref(cfg), rows)
        self.ctx = Context(l.gd_gpt_params_bytes(C.byref(cfg)), l.gd_gpt_state_bytes(C.byref(cfg)),
                           scratch_slot_bytes, data_slot_bytes=max(1 << 20, 16 * rows + (1 << 16)))
        h = _vp()
        st = l.gd_gpt_decoder_create(self.ctx.handle, C.byref(cfg), C.byref(h))
        if st != GD_OK:
            msg = self.ctx.error()
            self.ctx.close()
            raise GdError(st, f"gd_gpt_decoder_create [{msg}]")
        self.handle = h.value

    def close(self):
        if getattr(self, "handle", None):
            lib().gd_gpt_decoder_destroy(self.handle)
            self.handle = None
        if getattr(self, "ctx", None):
            self.ctx.close()
            self.ctx = None

    def tensor(self, name, layer=0):
        p = lib().gd_gpt_decoder_tensor(self.handle, name.encode(), layer)
        if not p:
            raise KeyError(name)
        return p.contents

    def read_tensor(self, name, layer=0):
        st, a = self.ctx.read(self.tensor(name, layer), np.float16)
        self.ctx.check(st, "gd_tensor_read")
        return a

    def load_checkpoint(self, path, strict=True):
        """Weights from a .gdckpt file the reference wrote for its gpt_lm example (strict as in the reference's
        gd_module_load_options)."""
        self.ctx.check(lib().gd_gpt_decoder_load_checkpoint(self.handle, os.fsencode(path), 1 if strict else 0),
                       "gd_gpt_decoder_load_checkpoint")

    def write_tensor(self, name, layer, array):
        self.ctx.check(self.ctx.write(self.tensor(name, layer), array), "gd_tensor_write")

    @property
    def positions(self):
        p = lib().gd_gpt_decoder_positions(self.handle)
        return np.ctypeslib.as_array(p, shape=(self.cfg.batch,))

    def _outputs(self, want_logits):
        B, V = self.cfg.batch, self.cfg.vocab
        nxt, gap = np.empty(B, np.int32), np.empty(B, np.float32)
        logits = np.empty((B, V), np.float16) if want_logits else None
        return nxt, gap, logits

    def prefill(self, ids, cu, want_logits=True):
        ids, cu = np.ascontiguousarray(ids, np.int32), np.ascontiguousarray(cu, np.int32)
        nxt, gap, logits = self._outputs(want_logits)
        st = lib().gd_gpt_decoder_prefill(self.handle, ids.ctypes.data_as(_vp), cu.ctypes.data_as(_vp),
                                          nxt.ctypes.data_as(_vp), gap.ctypes.data_as(_vp),
                                          logits.ctypes.data_as(_vp) if want_logits else None)
        self.ctx.check(st, "gd_gpt_decoder_prefill")
        return logits, nxt, gap

    def step(self, ids, want_logits=True):
        ids = np.ascontiguousarray(ids, np.int32)
        nxt, gap, logits = self._outputs(want_logits)
        st = lib().gd_gpt_decoder_step(self.handle, ids.ctypes.data_as(_vp), nxt.ctypes.data_as(_vp),
                                       gap.ctypes.data_as(_vp), logits.ctypes.data_as(_vp) if want_logits else None)
        self.ctx.check(st, "gd_gpt_decoder_step")
        return logits, nxt, gap

    def run_resident(self, first_ids, n_steps):
        first = np.ascontiguousarray(first_ids, np.int32)
        ids = np.empty((n_steps, self.cfg.batch), np.int32)
        gaps = np.empty((n_steps, self.cfg.batch), np.float32)
        ms = C.c_float()
        st = lib().gd_gpt_decoder_run_resident(self.handle, first.ctypes.data_as(_vp), n_steps,
                                               ids.ctypes.data_as(_vp), gaps.ctypes.data_as(_vp), C.byref(ms))
        self.ctx.check(st, "gd_gpt_decoder_run_resident")
        return ids, gaps, ms.value

    def generate(self, ids, cu, max_new, temperature=0.0, min_p=0.0, repetition_penalty=1.0, logits_softcap=0.0,
                 stop_token=-1, rng_state=0):
        """Packed prompts in, new tokens out (list of one int32 array per batch row): gd_gpt_decoder_generate."""
        ids, cu = np.ascontiguousarray(ids, np.int32), np.ascontiguousarray(cu, np.int32)
        s = GptSampling(temperature, min_p, repetition_penalty, logits_softcap, stop_token, rng_state)
        out = np.full((self.cfg.batch, max_new), -1, np.int32)
        counts = np.zeros(self.cfg.batch, np.int32)
        st = lib().gd_gpt_decoder_generate(self.handle, ids.ctypes.data_as(_vp), cu.ctypes.data_as(_vp), max_new,
                                           C.byref(s), out.ctypes.data_as(_vp), counts.ctypes.data_as(_vp))
        self.ctx.check(st, "gd_gpt_decoder_generate")
        return [out[b, :counts[b]].copy() for b in range(self.cfg.batch)]

    def resident_begin(self, first_ids, max_steps, hold_positions=False, unfused=False, keep_logits=False):
        first = np.ascontiguousarray(first_ids, np.int32)
        flags = (1 if hold_positions else 0) | (2 if unfused else 0) | (4 if keep_logits else 0)
        self.ctx.check(lib().gd_gpt_decoder_resident_begin(self.handle, first.ctypes.data_as(_vp), max_steps, flags),
                       "gd_gpt_decoder_resident_begin")
        self._resident_max = max_steps  # only a session that opened sizes what resident_end downloads

    def resident_begin_sampled(self, ids, cu, max_picks, temperature, min_p=0.0, repetition_penalty=1.0,
                               logits_softcap=0.0, stop_token=-1, rng_state=0, hold_positions=False, unfused=False):
        ids, cu = np.ascontiguousarray(ids, np.int32), np.ascontiguousarray(cu, np.int32)
        s = GptSampling(temperature, min_p, repetition_penalty, logits_softcap, stop_token, rng_state)
        flags = (1 if hold_positions else 0) | (2 if unfused else 0)
        self.ctx.check(lib().gd_gpt_decoder_resident_begin_sampled(self.handle, ids.ctypes.data_as(_vp),
                                                                   cu.ctypes.data_as(_vp), max_picks, flags, C.byref(s)),
                       "gd_gpt_decoder_resident_begin_sampled")
        self._resident_max = max_picks

    def resident_run(self, n_steps):
        self.ctx.check(lib().gd_gpt_decoder_resident_run(self.handle, n_steps), "gd_gpt_decoder_resident_run")

    def resident_sync(self):
        self.ctx.check(lib().gd_gpt_decoder_resident_sync(self.handle), "gd_gpt_decoder_resident_sync")

    def resident_end(self):
        ids = np.empty((self._resident_max, self.cfg.batch), np.int32)
        gaps = np.empty((self._resident_max, self.cfg.batch), np.float32)
        done = C.c_int32()
        self.ctx.check(lib().gd_gpt_decoder_resident_end(self.handle, ids.ctypes.data_as(_vp), gaps.ctypes.data_as(_vp),
                                                         C.byref(done)), "gd_gpt_decoder_resident_end")
        return ids[:done.value], gaps[:done.value]


def view_of(t):
    """gd_backend_tensor_view of a contiguous gd_tensor (what the operator front ends build)."""
    from . import TensorView
    v = TensorView()
    v.buffer, v.offset, v.dtype, v.rank = t.storage.buffer, t.storage.offset + t.view_offset, t.dtype, t.rank
    n, st = 1, 1
    for d in range(t.rank - 1, -1, -1):
        v.shape[d], v.strides[d] = t.shape[d], st
        st *= t.shape[d]
    v.count = st
    return v


_CKPT_NUMPY = {1: np.float16, 3: np.float32, 4: np.int32, 5: np.uint8, 6: np.uint16}


class Checkpoint:
    """Read-only view of a .gdckpt file (gd_checkpoint_*): directory entries, metadata, raw tensor bytes."""

    def __init__(self, path):
        self.handle = _vp()
        st = lib().gd_checkpoint_open(os.fsencode(path), C.byref(self.handle))
        if st != GD_OK:
            self.handle = None
            raise GdError(st, f"gd_checkpoint_open({path})")
        self.path = path

    def close(self):
        if getattr(self, "handle", None):
            lib().gd_checkpoint_close(self.handle)
            self.handle = None

    __del__ = close

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __len__(self):
        return lib().gd_checkpoint_count(self.handle)

    def entries(self):
        return [lib().gd_checkpoint_entry_at(self.handle, i).contents for i in range(len(self))]

    def paths(self):
        return [e.path.decode() for e in self.entries()]

    def metadata(self):
        blob, n = _vp(), C.c_size_t()
        st = lib().gd_checkpoint_read_metadata(os.fsencode(self.path), C.byref(blob), C.byref(n))
        if st != GD_OK:
            raise GdError(st, "gd_checkpoint_read_metadata")
        try:
            return C.string_at(blob, n.value)
        finally:
            _libc_free(blob)

    def read(self, path):
        """The tensor stored under `path` as a numpy array (BF16 comes back as its uint16 bits)."""
        p = lib().gd_checkpoint_find(self.handle, path.encode())
        if not p:
            raise KeyError(path)
        e = p.contents
        raw = np.empty(e.nbytes, np.uint8)
        st = lib().gd_checkpoint_read(self.handle, p, 0, raw.ctypes.data_as(_vp), e.nbytes)
        if st != GD_OK:
            raise GdError(st, f"gd_checkpoint_read({path})")
        dtype = np.uint16 if e.dtype == 2 else _CKPT_NUMPY[e.dtype]
        return raw.view(dtype).reshape([e.shape[i] for i in range(e.rank)])


def _libc_free(ptr):
    libc = C.CDLL(None)
    libc.free.argtypes = [_vp]
    libc.free.restype = None
    libc.free(ptr)
