"""Python host side of the MI355X backend for the gradients.c decode path.

A thin ctypes binding of ``libgradients_hip.so`` (the C-ABI declared in
``include/gd_backend_hip.h``): device buffers, tensor/matrix views and one
method per ``gd_backend_*`` operator, with the reference's names and argument
meaning.  There is no CPU fallback: importing works anywhere, but creating a
:class:`Backend` raises when the library is missing or no HIP device answers.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgradients_hip.so")
CSRC = os.path.join(_HERE, "csrc")

# gd_status (reference include/gradients/status.h:8-19)
GD_OK = 0
STATUS_NAMES = {0: "GD_OK", -1: "GD_ERR_INVALID_ARGUMENT", -2: "GD_ERR_OUT_OF_MEMORY", -3: "GD_ERR_FROZEN",
                -4: "GD_ERR_BUSY", -5: "GD_ERR_BAD_STATE", -6: "GD_ERR_UNSUPPORTED", -7: "GD_ERR_INTERNAL",
                -8: "GD_ERR_NOT_IMPLEMENTED", -9: "GD_ERR_IO"}
INVALID_ARGUMENT, BAD_STATE, UNSUPPORTED = -1, -5, -6

# dtype codes (reference include/gradients/tensor.h:49-57)
F16, BF16, F32, I32, U8, U16 = 1, 2, 3, 4, 5, 6
_NP_DTYPE = {F16: np.float16, F32: np.float32, I32: np.int32, U8: np.uint8, U16: np.uint16}
_CODE_OF = {np.dtype(np.float16): F16, np.dtype(np.float32): F32, np.dtype(np.int32): I32,
            np.dtype(np.uint8): U8, np.dtype(np.uint16): U16}


class GdError(RuntimeError):
    def __init__(self, status, what):
        super().__init__(f"{what}: {STATUS_NAMES.get(status, status)}")
        self.status = status


class TensorView(C.Structure):  # gd_backend_tensor_view
    _fields_ = [("buffer", C.c_void_p), ("offset", C.c_size_t), ("count", C.c_size_t), ("dtype", C.c_uint32),
                ("rank", C.c_uint32), ("shape", C.c_int64 * 8), ("strides", C.c_int64 * 8)]


class MatrixView(C.Structure):  # gd_backend_matrix_view
    _fields_ = [("buffer", C.c_void_p), ("offset", C.c_size_t), ("rows", C.c_uint32), ("cols", C.c_uint32),
                ("row_bytes", C.c_size_t), ("dtype", C.c_uint32)]


class VectorView(C.Structure):  # gd_backend_vector_view
    _fields_ = [("buffer", C.c_void_p), ("offset", C.c_size_t), ("length", C.c_uint32), ("dtype", C.c_uint32)]


class EmbeddingArgs(C.Structure):
    _fields_ = [("ids_count", C.c_uint64), ("vocab", C.c_uint64), ("dim", C.c_uint64)]


class RmsNormArgs(C.Structure):
    _fields_ = [("rows", C.c_uint64), ("cols", C.c_uint64), ("row_blocks", C.c_uint64), ("eps", C.c_float),
                ("simdgroups", C.c_uint32), ("wgrad_simdgroups", C.c_uint32), ("wgrad_row_block", C.c_uint32),
                ("reserved0", C.c_uint32)]


class RopeArgs(C.Structure):
    _fields_ = [("theta", C.c_float), ("n_dims", C.c_uint32), ("interleaved", C.c_uint32)]


class SdpaVarlenArgs(C.Structure):
    _fields_ = [("scale", C.c_float), ("causal", C.c_uint32), ("sliding_window", C.c_uint32),
                ("prefix_len", C.c_uint32), ("max_seqlen", C.c_uint32), ("use_forward_stats", C.c_uint32)]


class SdpaDecodeArgs(C.Structure):
    _fields_ = [("scale", C.c_float), ("sliding_window", C.c_uint32), ("prefix_len", C.c_uint32),
                ("cache_pos", C.c_int32)]


class FusedLinearArgs(C.Structure):
    _fields_ = [("w_is_nk", C.c_uint32), ("bias_mode", C.c_uint32), ("prologue", C.c_uint32), ("eps", C.c_float),
                ("epilogue", C.c_uint32)]


class MinimaxArgs(C.Structure):  # gd_backend_minimax_m3_sparse_args
    _fields_ = [("scale", C.c_float), ("block_size", C.c_uint32), ("topk", C.c_uint32), ("init_blocks", C.c_uint32),
                ("local_blocks", C.c_uint32), ("max_seqlen", C.c_uint32)]


class SampleArgs(C.Structure):  # gd_backend_sample_args
    _fields_ = [("temperature", C.c_float), ("min_p", C.c_float), ("repetition_penalty", C.c_float),
                ("logits_softcap", C.c_float), ("stop_token", C.c_int32), ("pos_delta", C.c_int32)]


class SampleTensors(C.Structure):  # gd_backend_sample_tensors
    _names = ("history", "hist_len", "finished", "state", "work", "ids", "positions", "step_counters", "out_ids",
              "table", "next_x")
    _fields_ = [(n, C.POINTER(TensorView)) for n in _names]


class ConcatArgs(C.Structure):
    _fields_ = [("count", C.c_uint64), ("inner", C.c_uint64), ("slice_axis", C.c_uint64), ("full_axis", C.c_uint64),
                ("axis_offset", C.c_uint64)]


class KvAppendArgs(C.Structure):
    _fields_ = [("cache_pos", C.c_int32)]


class Fence(C.Structure):
    _fields_ = [("handle", C.c_void_p)]


def build(force=False):
    """Compile the backend for gfx950 with hipcc (cross-compiles without a GPU)."""
    args = ["make", "-C", CSRC, "-j8"] + (["-B"] if force else [])
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)
    return LIB_PATH


_lib = None

_TV, _MV, _VV, _vp = C.POINTER(TensorView), C.POINTER(MatrixView), C.POINTER(VectorView), C.c_void_p

# name -> argtypes (restype is gd_status = int unless listed in _OTHER_RESTYPE)
_SIGNATURES = {
    "gd_backend_create_default": [C.POINTER(_vp)],
    "gd_backend_buffer_create": [_vp, C.c_size_t, C.POINTER(_vp)],
    "gd_backend_scope_begin": [_vp],
    "gd_backend_flush": [_vp],
    "gd_backend_upload": [_vp, _vp, C.c_size_t, _vp, C.c_size_t],
    "gd_backend_download": [_vp, _vp, C.c_size_t, _vp, C.c_size_t],
    "gd_backend_fill": [_vp, _vp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint32],
    "gd_backend_record_fence": [_vp, C.POINTER(Fence)],
    "gd_backend_fence_wait": [C.POINTER(Fence)],
    "gd_backend_embedding_forward": [_vp, _TV, _TV, _TV, C.POINTER(EmbeddingArgs)],
    "gd_backend_rms_norm_forward": [_vp, _TV, _TV, _TV, C.POINTER(RmsNormArgs)],
    "gd_backend_matmul": [_vp, _MV, _MV, _MV],
    "gd_backend_matmul_nt": [_vp, _MV, _MV, _MV],
    "gd_backend_linear": [_vp, _MV, _MV, _VV, _MV],
    "gd_backend_add": [_vp, _TV, _TV, _TV],
    "gd_backend_qkv_split_rope_forward": [_vp, _TV, _TV, _TV, _TV, _TV, C.c_uint32, C.c_uint32, C.POINTER(RopeArgs)],
    "gd_backend_swiglu_split_forward": [_vp, _TV, _TV],
    "gd_backend_sdpa_varlen": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, C.POINTER(SdpaVarlenArgs)],
    "gd_backend_sdpa_varlen_cached": [_vp, _TV, _TV, _TV, _TV, _TV, C.POINTER(SdpaVarlenArgs)],
    "gd_backend_sdpa_decode": [_vp, _TV, _TV, _TV, _TV, _TV, C.POINTER(SdpaDecodeArgs)],
    "gd_backend_sdpa_decode_at": [_vp, _TV, _TV, _TV, _TV, C.POINTER(SdpaDecodeArgs)],
    "gd_backend_sdpa_decode_positions": [_vp, _TV, _TV, _TV, _TV, _TV, C.POINTER(SdpaDecodeArgs)],
    "gd_backend_sdpa_decode_positions_noalloc": [_vp, _TV, _TV, _TV, _TV, _TV, C.POINTER(SdpaDecodeArgs)],
    "gd_backend_kv_cache_append_at": [_vp, _TV, _TV, _TV, _TV, C.POINTER(KvAppendArgs)],
    "gd_backend_kv_cache_append_positions": [_vp, _TV, _TV, _TV, _TV, _TV, C.POINTER(KvAppendArgs)],
    "gd_backend_kv_cache_append_packed": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, C.POINTER(KvAppendArgs)],
    "gd_backend_argmax_rows": [_vp, _TV, _TV, _TV],
    "gd_backend_swiglu_split_linear": [_vp, _MV, _MV, _VV, _MV],
    "gd_backend_linear_nt": [_vp, _MV, _MV, _VV, _MV],
    "gd_backend_fused_linear": [_vp, _MV, _MV, _VV, _MV, _VV, _MV, C.POINTER(FusedLinearArgs)],
    "gd_backend_qkv_rope_append": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, C.c_uint32, C.c_uint32, C.POINTER(RopeArgs)],
    "gd_backend_qkv_rope_append_packed": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, _TV, _TV, _TV, C.c_uint32, C.c_uint32,
                                          C.POINTER(RopeArgs)],
    "gd_backend_rope_table_packed": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, C.c_uint32, C.c_uint32, C.POINTER(RopeArgs)],
    "gd_backend_linear_qkv_rope_packed": [_vp, _MV, _MV, _VV, _TV, _TV, _TV, _TV, _TV, _TV, _MV, C.c_uint32, C.c_uint32,
                                          C.c_uint32],
    "gd_backend_rand_uniform": [_vp, _vp, C.c_size_t, C.c_size_t, C.c_uint32, C.c_uint64, C.c_float, C.c_float],
    "gd_backend_concat_to_full": [_vp, _TV, _TV, C.POINTER(ConcatArgs)],
    "gd_backend_gather_rows": [_vp, _TV, _TV, _TV],
    "gd_backend_add_scalar_i32": [_vp, _TV, _TV, C.c_int32],
    "gd_backend_decode_advance": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, _TV, C.c_int32],
    "gd_backend_fused_qkv_rope_append": [_vp, _MV, _MV, _VV, _VV, _TV, _TV, _TV, _TV, _TV, C.c_uint32, C.c_uint32,
                                         C.POINTER(RopeArgs), C.POINTER(FusedLinearArgs)],
    "gd_backend_argmax_advance": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, C.c_int32, _TV, _TV],
    "gd_backend_sample_advance": [_vp, _TV, C.POINTER(SampleTensors), C.POINTER(SampleArgs)],
    "gd_backend_minimax_m3_index_topk": [_vp, _TV, _TV, _TV, _TV, C.POINTER(MinimaxArgs)],
    "gd_backend_minimax_m3_sparse_attention": [_vp, _TV, _TV, _TV, _TV, _TV, _TV, C.POINTER(MinimaxArgs)],
    "gd_backend_copy": [_vp, _vp, C.c_size_t, _vp, C.c_size_t, C.c_size_t],
    "gd_backend_timer_create": [_vp, C.POINTER(_vp)],
    "gd_backend_timer_start": [_vp],
    "gd_backend_timer_stop": [_vp],
    "gd_backend_timer_elapsed_ms": [_vp, C.POINTER(C.c_float)],
    "gd_backend_graph_begin_capture": [_vp],
    "gd_backend_graph_end_capture": [_vp, C.POINTER(_vp)],
    "gd_backend_graph_launch": [_vp, _vp],
    "gd_backend_device_info": [_vp, C.c_char_p, C.c_size_t, C.POINTER(C.c_int32), C.POINTER(C.c_uint64)],
    "gd_backend_set_tunable": [_vp, C.c_char_p, C.c_int64],
    "gd_backend_sdpa_decode_last_kernel": [_vp, C.c_char_p, C.c_size_t],
    "gd_backend_linear_last_kernel": [_vp, C.c_char_p, C.c_size_t],
}
_OTHER_RESTYPE = {
    "gd_backend_destroy": (None, [_vp]),
    "gd_backend_kind_query": (C.c_int, [_vp]),
    "gd_backend_name": (C.c_char_p, [_vp]),
    "gd_backend_buffer_destroy": (None, [_vp]),
    "gd_backend_buffer_nbytes": (C.c_size_t, [_vp]),
    "gd_backend_buffer_host_ptr": (_vp, [_vp]),
    "gd_backend_buffer_is_host_visible": (C.c_bool, [_vp]),
    "gd_backend_buffer_device_ptr": (_vp, [_vp]),
    "gd_backend_fence_destroy": (None, [C.POINTER(Fence)]),
    "gd_backend_fence_is_complete": (C.c_bool, [C.POINTER(Fence)]),
    "gd_backend_timer_destroy": (None, [_vp]),
    "gd_backend_sample_state_count": (C.c_size_t, [C.c_uint32]),
    "gd_backend_sample_work_count": (C.c_size_t, [C.c_uint32, C.c_uint32]),
    "gd_backend_graph_destroy": (None, [_vp]),
}
EXPORTED_SYMBOLS = sorted(list(_SIGNATURES) + list(_OTHER_RESTYPE))


def lib():
    """Load the built library.  Raises when it has not been built (call build() first)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with __graft_entry__.build() "
                               "(there is no CPU fallback)")
        l = C.CDLL(LIB_PATH)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = C.c_int
            fn.argtypes = argtypes
        for name, (restype, argtypes) in _OTHER_RESTYPE.items():
            fn = getattr(l, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = l
    return _lib


def _check(status, what):
    if status != GD_OK:
        raise GdError(status, what)


class Tensor:
    """A contiguous region of a device buffer plus its descriptor (what gd_tensor is to the core)."""

    def __init__(self, buffer, offset, shape, dtype):
        self.buffer, self.offset, self.shape, self.dtype = buffer, int(offset), tuple(int(s) for s in shape), dtype
        self.count = int(np.prod(self.shape)) if self.shape else 1
        self.itemsize = np.dtype(_NP_DTYPE[dtype]).itemsize
        self.nbytes = self.count * self.itemsize

    def view(self, shape=None, strides=None):
        shape = self.shape if shape is None else tuple(shape)
        v = TensorView()
        v.buffer, v.offset, v.dtype, v.rank = self.buffer.handle, self.offset, self.dtype, len(shape)
        v.count = int(np.prod(shape)) if shape else 1
        st = 1
        for d in range(len(shape) - 1, -1, -1):
            v.shape[d] = shape[d]
            v.strides[d] = st if strides is None else strides[d]
            st *= shape[d]
        return v

    def matrix(self, rows=None, cols=None, row_elems=None):
        cols = self.shape[-1] if cols is None else cols
        rows = self.count // self.shape[-1] if rows is None else rows
        m = MatrixView()
        m.buffer, m.offset, m.rows, m.cols, m.dtype = self.buffer.handle, self.offset, rows, cols, self.dtype
        m.row_bytes = (self.shape[-1] if row_elems is None else row_elems) * self.itemsize
        return m

    def vector(self):
        v = VectorView()
        v.buffer, v.offset, v.length, v.dtype = self.buffer.handle, self.offset, self.count, self.dtype
        return v

    def reshape(self, *shape):
        assert int(np.prod(shape)) == self.count
        return Tensor(self.buffer, self.offset, shape, self.dtype)

    def rows(self, start, n):
        """Leading-dimension slice (shares storage), like gd_tensor_slice on dim 0."""
        inner = self.count // self.shape[0]
        return Tensor(self.buffer, self.offset + start * inner * self.itemsize, (n,) + self.shape[1:], self.dtype)

    def write(self, array):
        a = np.ascontiguousarray(array, dtype=_NP_DTYPE[self.dtype])
        assert a.size == self.count, (a.shape, self.shape)
        self.buffer.upload(self.offset, a)
        return self

    def read(self):
        out = np.empty(self.shape, _NP_DTYPE[self.dtype])
        self.buffer.download(self.offset, out)
        return out


class Buffer:
    """gd_backend_buffer with a bump allocator (256-byte alignment, the core's default)."""

    def __init__(self, backend, nbytes):
        self.backend, self.nbytes, self._top = backend, int(nbytes), 0
        h = _vp()
        _check(lib().gd_backend_buffer_create(backend.handle, self.nbytes, C.byref(h)), "gd_backend_buffer_create")
        self.handle = h.value

    def close(self):
        if self.handle:
            lib().gd_backend_buffer_destroy(self.handle)
            self.handle = None

    def reset(self):
        self._top = 0

    def alloc(self, shape, dtype, align=256):
        off = (self._top + align - 1) // align * align
        t = Tensor(self, off, shape, dtype)
        if off + t.nbytes > self.nbytes:
            raise GdError(-2, "arena exhausted")
        self._top = off + t.nbytes
        return t

    def from_numpy(self, array):
        a = np.ascontiguousarray(array)
        return self.alloc(a.shape, _CODE_OF[a.dtype]).write(a)

    def upload(self, offset, array):
        _check(lib().gd_backend_upload(self.backend.handle, self.handle, offset, array.ctypes.data_as(_vp),
                                       array.nbytes), "gd_backend_upload")

    def download(self, offset, out):
        _check(lib().gd_backend_download(self.backend.handle, self.handle, offset, out.ctypes.data_as(_vp),
                                         out.nbytes), "gd_backend_download")


class Timer:
    def __init__(self, backend):
        h = _vp()
        _check(lib().gd_backend_timer_create(backend.handle, C.byref(h)), "gd_backend_timer_create")
        self.handle = h.value

    def start(self):
        _check(lib().gd_backend_timer_start(self.handle), "gd_backend_timer_start")

    def stop(self):
        _check(lib().gd_backend_timer_stop(self.handle), "gd_backend_timer_stop")

    def elapsed_ms(self):
        ms = C.c_float()
        _check(lib().gd_backend_timer_elapsed_ms(self.handle, C.byref(ms)), "gd_backend_timer_elapsed_ms")
        return ms.value

    def close(self):
        if self.handle:
            lib().gd_backend_timer_destroy(self.handle)
            self.handle = None


class Backend:
    """gd_backend: one HIP device, one stream.  Methods mirror the gd_backend_* operators."""

    def __init__(self, borrowed_handle=None):
        """Creates the default backend, or wraps the backend owned by a gd_context (borrowed)."""
        self._owned = borrowed_handle is None
        if self._owned:
            h = _vp()
            st = lib().gd_backend_create_default(C.byref(h))
            if st != GD_OK:
                raise GdError(st, "gd_backend_create_default (no HIP device? there is no CPU fallback)")
            self.handle = h.value
        else:
            self.handle = borrowed_handle
        self._buffers = []

    def close(self):
        for b in self._buffers:
            b.close()
        self._buffers = []
        if self.handle and self._owned:
            lib().gd_backend_destroy(self.handle)
        self.handle = None

    @property
    def name(self):
        return lib().gd_backend_name(self.handle).decode()

    def device_info(self):
        name = C.create_string_buffer(128)
        cus, mem = C.c_int32(), C.c_uint64()
        _check(lib().gd_backend_device_info(self.handle, name, 128, C.byref(cus), C.byref(mem)), "device_info")
        return name.value.decode(), cus.value, mem.value

    def set_tunable(self, name, value):
        _check(lib().gd_backend_set_tunable(self.handle, name.encode(), value), "gd_backend_set_tunable")

    def linear_last_kernel(self):
        out = C.create_string_buffer(32)
        _check(lib().gd_backend_linear_last_kernel(self.handle, out, 32), "gd_backend_linear_last_kernel")
        return out.value.decode()

    def sdpa_decode_last_kernel(self):
        out = C.create_string_buffer(160)
        _check(lib().gd_backend_sdpa_decode_last_kernel(self.handle, out, 160), "gd_backend_sdpa_decode_last_kernel")
        return out.value.decode()

    def buffer(self, nbytes):
        b = Buffer(self, nbytes)
        self._buffers.append(b)
        return b

    def free(self, buf):
        self._buffers.remove(buf)
        buf.close()

    # ---- scope ----
    def scope_begin(self):
        _check(lib().gd_backend_scope_begin(self.handle), "gd_backend_scope_begin")

    def record_fence(self):
        f = Fence()
        _check(lib().gd_backend_record_fence(self.handle, C.byref(f)), "gd_backend_record_fence")
        return f

    def fence_wait(self, fence, destroy=True):
        _check(lib().gd_backend_fence_wait(C.byref(fence)), "gd_backend_fence_wait")
        if destroy:
            lib().gd_backend_fence_destroy(C.byref(fence))

    def flush(self):
        _check(lib().gd_backend_flush(self.handle), "gd_backend_flush")

    def fill(self, tensor, pattern):
        _check(lib().gd_backend_fill(self.handle, tensor.buffer.handle, tensor.offset, tensor.count,
                                     tensor.itemsize, pattern), "gd_backend_fill")

    def rand_uniform(self, tensor, seed, low, high):
        _check(lib().gd_backend_rand_uniform(self.handle, tensor.buffer.handle, tensor.offset, tensor.count,
                                             tensor.dtype, seed, low, high), "gd_backend_rand_uniform")

    def call(self, name, *args):
        """Raw status of a gd_backend_* call (for error-path tests)."""
        return getattr(lib(), name)(self.handle, *args)

    # ---- operators (raise on a non-OK status) ----
    def embedding_forward(self, table, ids, out):
        a = EmbeddingArgs(ids.count, table.shape[0], table.shape[1])
        _check(self.call("gd_backend_embedding_forward", table.view(), ids.view(), out.view(), C.byref(a)),
               "gd_backend_embedding_forward")

    def rms_norm_forward(self, x, w, out, eps):
        a = RmsNormArgs(rows=x.count // x.shape[-1], cols=x.shape[-1], eps=eps)
        _check(self.call("gd_backend_rms_norm_forward", x.view(), w.view(), out.view(), C.byref(a)),
               "gd_backend_rms_norm_forward")

    def matmul(self, x, w, y):
        _check(self.call("gd_backend_matmul", x.matrix(), w.matrix(), y.matrix()), "gd_backend_matmul")

    def matmul_nt(self, x, w, y):
        _check(self.call("gd_backend_matmul_nt", x.matrix(), w.matrix(), y.matrix()), "gd_backend_matmul_nt")

    def linear(self, x, w, bias, y):
        _check(self.call("gd_backend_linear", x.matrix(), w.matrix(), bias.vector(), y.matrix()), "gd_backend_linear")

    def linear_nt(self, x, w, bias, y):
        _check(self.call("gd_backend_linear_nt", x.matrix(), w.matrix(), bias.vector() if bias else None,
                         y.matrix()), "gd_backend_linear_nt")

    def swiglu_split_linear(self, x12, w, bias, y):
        _check(self.call("gd_backend_swiglu_split_linear", x12.matrix(), w.matrix(),
                         bias.vector() if bias else None, y.matrix()), "gd_backend_swiglu_split_linear")

    def fused_linear(self, x, w, bias, residual, norm_weight, y, w_is_nk, bias_mode, prologue, eps=0.0, epilogue=0):
        a = FusedLinearArgs(int(w_is_nk), bias_mode, prologue, eps, epilogue)
        _check(self.call("gd_backend_fused_linear", x.matrix(), w.matrix(), bias.vector() if bias else None,
                         residual.matrix() if residual else None, norm_weight.vector() if norm_weight else None,
                         y.matrix(), C.byref(a)), "gd_backend_fused_linear")

    def add(self, x, y, out):
        _check(self.call("gd_backend_add", x.view(), y.view(), out.view()), "gd_backend_add")

    def qkv_split_rope_forward(self, qkv, pos, q, k, v, n_heads, head_dim, theta=10000.0, interleaved=False):
        a = RopeArgs(theta, head_dim, int(interleaved))
        _check(self.call("gd_backend_qkv_split_rope_forward", qkv.view(), pos.view(), q.view(), k.view(), v.view(),
                         n_heads, head_dim, C.byref(a)), "gd_backend_qkv_split_rope_forward")

    def qkv_rope_append(self, qkv, pos, cache_pos, q, k_cache, v_cache, n_heads, head_dim, theta=10000.0):
        a = RopeArgs(theta, head_dim, 0)
        _check(self.call("gd_backend_qkv_rope_append", qkv.view(), pos.view(), cache_pos.view(), q.view(),
                         k_cache.view(), v_cache.view(), n_heads, head_dim, C.byref(a)), "gd_backend_qkv_rope_append")

    def qkv_rope_append_packed(self, qkv, pos, cache_pos, cu, q, k, v, k_cache, v_cache, n_heads, head_dim, theta=10000.0):
        a = RopeArgs(theta, head_dim, 0)
        _check(self.call("gd_backend_qkv_rope_append_packed", qkv.view(), pos.view(), cache_pos.view(), cu.view(), q.view(),
                         k.view() if k is not None else None, v.view() if v is not None else None, k_cache.view(),
                         v_cache.view(), n_heads, head_dim, C.byref(a)),
               "gd_backend_qkv_rope_append_packed")

    def rope_table_packed(self, pos, cache_pos, cu, cos_rows, sin_rows, cache_rows, head_dim, tmax, theta=10000.0):
        a = RopeArgs(theta, head_dim, 0)
        _check(self.call("gd_backend_rope_table_packed", pos.view(), cache_pos.view(), cu.view(), cos_rows.view(),
                         sin_rows.view(), cache_rows.view(), head_dim, tmax, C.byref(a)), "gd_backend_rope_table_packed")

    def linear_qkv_rope_packed(self, x, w, bias, cos_rows, sin_rows, cache_rows, q, k_cache, v_cache, work, n_heads,
                               head_dim, bias_mode):
        _check(self.call("gd_backend_linear_qkv_rope_packed", x.matrix(), w.matrix(), bias.vector() if bias else None,
                         cos_rows.view(), sin_rows.view(), cache_rows.view(), q.view(), k_cache.view(), v_cache.view(),
                         work.matrix(), n_heads, head_dim, bias_mode), "gd_backend_linear_qkv_rope_packed")

    def fused_qkv_rope_append(self, x, w, bias, norm_weight, pos, cache_pos, q, k_cache, v_cache, n_heads, head_dim,
                              bias_mode, prologue, eps=0.0, theta=10000.0):
        ra, fa = RopeArgs(theta, head_dim, 0), FusedLinearArgs(1, bias_mode, prologue, eps, 0)
        _check(self.call("gd_backend_fused_qkv_rope_append", x.matrix(), w.matrix(), bias.vector() if bias else None,
                         norm_weight.vector() if norm_weight else None, pos.view(), cache_pos.view(), q.view(),
                         k_cache.view(), v_cache.view(), n_heads, head_dim, C.byref(ra), C.byref(fa)),
               "gd_backend_fused_qkv_rope_append")

    def swiglu_split_forward(self, x12, out):
        _check(self.call("gd_backend_swiglu_split_forward", x12.view(), out.view()), "gd_backend_swiglu_split_forward")

    def sdpa_varlen(self, q, k, v, cu, out, scale, causal=True, window=0, prefix=0, max_seqlen=0):
        a = SdpaVarlenArgs(scale, int(causal), window, prefix, max_seqlen, 0)
        _check(self.call("gd_backend_sdpa_varlen", q.view(), k.view(), v.view(), cu.view(), out.view(), None,
                         C.byref(a)), "gd_backend_sdpa_varlen")

    def sdpa_varlen_cached(self, q, k_cache, v_cache, cu, out, scale, causal=True, window=0, prefix=0, max_seqlen=0):
        a = SdpaVarlenArgs(scale, int(causal), window, prefix, max_seqlen, 0)
        _check(self.call("gd_backend_sdpa_varlen_cached", q.view(), k_cache.view(), v_cache.view(), cu.view(), out.view(),
                         C.byref(a)), "gd_backend_sdpa_varlen_cached")

    def sdpa_decode(self, q, k, v, pos, out, scale, window=0, prefix=0):
        a = SdpaDecodeArgs(scale, window, prefix, 0)
        _check(self.call("gd_backend_sdpa_decode", q.view(), k.view(), v.view(), pos.view(()), out.view(),
                         C.byref(a)), "gd_backend_sdpa_decode")

    def sdpa_decode_at(self, q, k, v, cache_pos, out, scale, window=0, prefix=0):
        a = SdpaDecodeArgs(scale, window, prefix, cache_pos)
        _check(self.call("gd_backend_sdpa_decode_at", q.view(), k.view(), v.view(), out.view(), C.byref(a)),
               "gd_backend_sdpa_decode_at")

    def sdpa_decode_positions(self, q, k, v, pos, out, scale, window=0, prefix=0):
        a = SdpaDecodeArgs(scale, window, prefix, 0)
        _check(self.call("gd_backend_sdpa_decode_positions", q.view(), k.view(), v.view(), pos.view(), out.view(),
                         C.byref(a)), "gd_backend_sdpa_decode_positions")

    def sdpa_decode_positions_noalloc(self, q, k, v, pos, out, scale, window=0, prefix=0):
        a = SdpaDecodeArgs(scale, window, prefix, 0)
        _check(self.call("gd_backend_sdpa_decode_positions_noalloc", q.view(), k.view(), v.view(), pos.view(),
                         out.view(), C.byref(a)), "gd_backend_sdpa_decode_positions_noalloc")

    def kv_cache_append_at(self, k_cache, v_cache, cache_pos, k_new, v_new):
        a = KvAppendArgs(cache_pos)
        _check(self.call("gd_backend_kv_cache_append_at", k_cache.view(), v_cache.view(), k_new.view(), v_new.view(),
                         C.byref(a)), "gd_backend_kv_cache_append_at")

    def kv_cache_append_positions(self, k_cache, v_cache, pos, k_new, v_new):
        a = KvAppendArgs(0)
        _check(self.call("gd_backend_kv_cache_append_positions", k_cache.view(), v_cache.view(), pos.view(),
                         k_new.view(), v_new.view(), C.byref(a)), "gd_backend_kv_cache_append_positions")

    def kv_cache_append_packed(self, k_cache, v_cache, pos, cu, k_new, v_new):
        a = KvAppendArgs(0)
        _check(self.call("gd_backend_kv_cache_append_packed", k_cache.view(), v_cache.view(), pos.view(), cu.view(),
                         k_new.view(), v_new.view(), C.byref(a)), "gd_backend_kv_cache_append_packed")

    def argmax_rows(self, logits, ids, gap=None):
        _check(self.call("gd_backend_argmax_rows", logits.view(), ids.view(), gap.view() if gap else None),
               "gd_backend_argmax_rows")

    def sample_advance(self, logits, tensors, temperature, min_p=0.0, repetition_penalty=1.0, logits_softcap=0.0,
                       stop_token=-1, pos_delta=1):
        """tensors: dict of Tensor by the field names of gd_backend_sample_tensors (table / next_x optional)."""
        views = {n: tensors[n].view() for n in SampleTensors._names if tensors.get(n) is not None}
        t = SampleTensors(**{n: C.pointer(v) for n, v in views.items()})
        a = SampleArgs(temperature, min_p, repetition_penalty, logits_softcap, stop_token, pos_delta)
        st = self.call("gd_backend_sample_advance", logits.view(), C.byref(t), C.byref(a))
        _check(st, "gd_backend_sample_advance")

    def minimax_m3_index_topk(self, q, k, cu, topk_idx, block, init_blocks=1, local_blocks=1, max_seqlen=None):
        a = MinimaxArgs(1.0, block, topk_idx.shape[2], init_blocks, local_blocks, max_seqlen or q.shape[0])
        _check(self.call("gd_backend_minimax_m3_index_topk", q.view(), k.view(), cu.view(), topk_idx.view(), C.byref(a)),
               "gd_backend_minimax_m3_index_topk")

    def minimax_m3_sparse_attention(self, q, k, v, cu, topk_idx, out, block, scale, max_seqlen=None):
        a = MinimaxArgs(scale, block, topk_idx.shape[2], 0, 0, max_seqlen or q.shape[0])
        _check(self.call("gd_backend_minimax_m3_sparse_attention", q.view(), k.view(), v.view(), cu.view(),
                         topk_idx.view(), out.view(), C.byref(a)), "gd_backend_minimax_m3_sparse_attention")

    @staticmethod
    def sample_work_count(rows, cols):
        return lib().gd_backend_sample_work_count(rows, cols)

    @staticmethod
    def sample_state_count(rows):
        return lib().gd_backend_sample_state_count(rows)

    def gather_rows(self, src, rows, out):
        _check(self.call("gd_backend_gather_rows", src.view(), rows.view(), out.view()), "gd_backend_gather_rows")

    def concat_to_full(self, src, dst, axis, axis_offset):
        """Place the contiguous slice `src` at `axis_offset` along `axis` of the contiguous `dst`."""
        inner = int(np.prod(src.shape[axis + 1:], dtype=np.int64))
        a = ConcatArgs(src.count, inner, src.shape[axis], dst.shape[axis], axis_offset)
        _check(self.call("gd_backend_concat_to_full", src.view(), dst.view(), C.byref(a)), "gd_backend_concat_to_full")

    def add_scalar_i32(self, src, dst, delta):
        _check(self.call("gd_backend_add_scalar_i32", src.view(), dst.view(), delta), "gd_backend_add_scalar_i32")

    # ---- graphs ----
    def graph_begin_capture(self):
        _check(lib().gd_backend_graph_begin_capture(self.handle), "gd_backend_graph_begin_capture")

    def graph_end_capture(self):
        g = _vp()
        _check(lib().gd_backend_graph_end_capture(self.handle, C.byref(g)), "gd_backend_graph_end_capture")
        return g.value

    def graph_launch(self, graph):
        _check(lib().gd_backend_graph_launch(self.handle, graph), "gd_backend_graph_launch")

    def graph_destroy(self, graph):
        lib().gd_backend_graph_destroy(graph)
