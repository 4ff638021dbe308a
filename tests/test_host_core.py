"""Host logic of the C core (context, arenas, ring slots, tensors, transfers) and of the operator front ends
(validation and status codes, output allocation), on the CPU.

The library under test is tests/host/libgradients_host.so: the product's own core/, ops/*/core_*.c and decoder/
sources linked with a device-less backend whose buffers are host memory and whose operator entry points compute
nothing (they count calls and return GD_OK).  What is asserted are the contracts the reference's own tests hold for
its core (tests/test_memory.c, test_tensor.c, test_transfer.c) and the status-code rules of its operator capsules
(src/ops/*/core_*.c), restated for this core.
"""
import ctypes as C

import numpy as np
import pytest

OK, INVALID, OOM, FROZEN, BAD_STATE, UNSUPPORTED = 0, -1, -2, -3, -5, -6
F16, F32, I32 = 1, 3, 4
PARAMS, STATE, SCRATCH, DATA = 0, 1, 2, 3
TRAIN, INFER = 1, 3


class RopeConfig(C.Structure):
    _fields_ = [("theta", C.c_float), ("n_dims", C.c_int32), ("interleaved", C.c_bool)]


class DecodeConfig(C.Structure):
    _fields_ = [("scale", C.c_float), ("sliding_window", C.c_int32), ("prefix_len", C.c_int32)]


class VarlenConfig(C.Structure):
    _fields_ = [("scale", C.c_float), ("causal", C.c_bool), ("sliding_window", C.c_int32), ("prefix_len", C.c_int32),
                ("max_seqlen", C.c_int32)]


@pytest.fixture()
def env(host):
    pkg, D = host
    l = D.lib()
    l.gd_null_backend_op_calls.restype = C.c_uint64
    l.gd_null_backend_last_op.restype = C.c_char_p
    l.gd_null_backend_fail_ops.argtypes = [C.c_int]
    ctx = D.Context(1 << 20, 1 << 20, 1 << 20, data_slot_bytes=1 << 16, scratch_slots=2, data_slots=2)
    yield D, l, ctx
    l.gd_debug_set_heap_guard(False)
    l.gd_null_backend_fail_ops(0)
    ctx.close()


def _t(D, ctx, arena, dtype, dims, zeros=False):
    st, t = ctx.empty(arena, dtype, dims, zeros=zeros)
    assert st == OK, ctx.error()
    return t


def _last(l):
    return l.gd_null_backend_last_op().decode()


# ---- arenas and ring slots (reference tests/test_memory.c:33-137) -------------------------------------------------

def test_allocation_rules_of_the_four_arenas(env):
    D, l, ctx = env
    span = D.Span()
    assert l.gd_alloc_scratch(ctx.handle, 64, 64, C.byref(span)) == BAD_STATE  # no step is open
    assert span.nbytes == 0 and not span.buffer and span.slot == -1               # failure clears the output
    assert l.gd_alloc_data(ctx.handle, 64, 64, C.byref(span)) == BAD_STATE
    assert l.gd_alloc_params(ctx.handle, 1000, 256, C.byref(span)) == OK
    assert span.arena == PARAMS and span.offset % 256 == 0 and span.nbytes == 1000 and span.slot == -1
    first_end = span.offset + span.nbytes
    assert l.gd_alloc_params(ctx.handle, 1 << 21, 256, C.byref(span)) == OOM     # larger than the arena
    assert span.nbytes == 0
    assert l.gd_alloc_params(ctx.handle, 8, 256, C.byref(span)) == OK
    assert span.offset == (first_end + 255) // 256 * 256                            # the failed request moved nothing
    assert l.gd_alloc_params(ctx.handle, 8, 48, C.byref(span)) == INVALID         # alignment not a power of two
    assert l.gd_context_seal_params(ctx.handle) == OK
    assert l.gd_alloc_params(ctx.handle, 8, 256, C.byref(span)) == FROZEN
    assert l.gd_alloc_state(ctx.handle, 8, 256, C.byref(span)) == OK              # state stays open


def test_ring_slots_rotate_and_bump_their_generation(env):
    D, l, ctx = env
    seen = []
    tensors = []
    for step in range(3):
        assert ctx.begin_step() == OK
        assert ctx.begin_step() == BAD_STATE  # a step is already open
        slot = l.gd_debug_current_ring_slot(ctx.handle, SCRATCH)
        gen = l.gd_debug_ring_slot_generation(ctx.handle, SCRATCH, slot)
        seen.append((slot, gen))
        tensors.append(_t(D, ctx, SCRATCH, F16, [4, 8]))
        assert l.gd_tensor_validate(ctx.handle, C.byref(tensors[-1])) == OK
        assert ctx.end_step() == OK
    assert ctx.end_step() == BAD_STATE
    assert [s for s, _ in seen] == [0, 1, 0]
    assert seen[2][1] == seen[0][1] + 1                       # slot 0 came back with a new generation
    assert l.gd_tensor_validate(ctx.handle, C.byref(tensors[1])) == OK      # slot 1 has not been reused
    assert l.gd_tensor_validate(ctx.handle, C.byref(tensors[0])) == BAD_STATE  # its storage was handed out again
    assert "stale" in ctx.error()
    out = np.empty((4, 8), np.float16)
    assert l.gd_tensor_read(ctx.handle, C.byref(tensors[0]), out.ctypes.data, out.nbytes) == BAD_STATE


def test_no_heap_allocation_inside_a_step(env):
    D, l, ctx = env
    w = _t(D, ctx, PARAMS, F16, [16, 8])
    assert ctx.begin_step() == OK
    before = l.gd_debug_heap_alloc_count()
    l.gd_debug_set_heap_guard(True)
    x = _t(D, ctx, SCRATCH, F16, [4, 8])
    y = D.GdTensor()
    assert l.gd_linear_transposed_weight(ctx.handle, C.byref(x), C.byref(w), None, C.byref(y)) == OK
    vals = np.arange(32, dtype=np.float32)
    assert l.gd_tensor_write_f32(ctx.handle, C.byref(x), vals.ctypes.data, 32) == OK
    back = np.empty(32, np.float32)
    assert l.gd_tensor_read_f32(ctx.handle, C.byref(x), back.ctypes.data, 32) == OK
    sl = D.GdTensor()
    assert l.gd_tensor_slice(ctx.handle, C.byref(x), 0, 1, 2, C.byref(sl)) == OK
    l.gd_debug_set_heap_guard(False)
    assert l.gd_debug_heap_alloc_count() == before
    assert np.array_equal(back, vals)
    assert ctx.end_step() == OK


# ---- tensors and transfers (reference tests/test_tensor.c, test_transfer.c) --------------------------------------

def test_tensor_descriptors_slices_and_fills(env):
    D, l, ctx = env
    t = _t(D, ctx, PARAMS, F16, [4, 8])
    assert (t.rank, t.shape[0], t.shape[1], t.strides[0], t.strides[1]) == (2, 4, 8, 8, 1)
    assert t.is_leaf and not t.is_view and t.storage.nbytes == 64 and t.id != 0
    z = _t(D, ctx, PARAMS, F32, [5], zeros=True)
    st, got = ctx.read(z, np.float32)
    assert st == OK and not got.any()
    ones = D.GdTensor()
    assert l.gd_tensor_ones(ctx.handle, PARAMS, F16, D.make_shape([3]), 256, C.byref(ones)) == OK
    assert np.array_equal(ctx.read(ones, np.float16)[1], np.ones(3, np.float16))
    bad = D.GdTensor()
    assert l.gd_tensor_empty(ctx.handle, PARAMS, F16, D.make_shape([4, 0]), 256, C.byref(bad)) == INVALID
    assert bad.storage.nbytes == 0
    rows = np.arange(32, dtype=np.float16).reshape(4, 8)
    assert ctx.write(t, rows) == OK
    v = D.GdTensor()
    assert l.gd_tensor_slice(ctx.handle, C.byref(t), 0, 1, 2, C.byref(v)) == OK
    assert v.is_view and v.view_offset == 16 and (v.shape[0], v.shape[1]) == (2, 8)
    assert v.storage.offset == t.storage.offset and l.gd_tensor_is_contiguous(C.byref(v))
    assert np.array_equal(ctx.read(v, np.float16)[1], rows[1:3])
    col = D.GdTensor()
    assert l.gd_tensor_slice(ctx.handle, C.byref(t), 1, 2, 3, C.byref(col)) == OK
    assert not l.gd_tensor_is_contiguous(C.byref(col))
    out = np.empty((4, 3), np.float16)
    assert l.gd_tensor_read(ctx.handle, C.byref(col), out.ctypes.data, out.nbytes) == UNSUPPORTED
    assert l.gd_tensor_slice(ctx.handle, C.byref(t), 1, 7, 4, C.byref(bad)) == INVALID
    assert bad.storage.nbytes == 0
    assert l.gd_tensor_slice(ctx.handle, C.byref(t), 2, 0, 1, C.byref(bad)) == INVALID


def test_f32_transfers_round_to_nearest_even(env):
    D, l, ctx = env
    rng = np.random.default_rng(3)
    vals = np.concatenate([rng.standard_normal(4000) * 10.0 ** rng.integers(-8, 5, 4000),
                           [0.0, -0.0, 65504.0, 65520.0, 1e-8, 2.0 ** -25, 2.0 ** -24, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11,
                            np.inf, -np.inf]]).astype(np.float32)
    t = _t(D, ctx, PARAMS, F16, [vals.size])
    assert l.gd_tensor_write_f32(ctx.handle, C.byref(t), vals.ctypes.data, vals.size) == OK
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16)
    st, got = ctx.read(t, np.float16)
    assert st == OK and np.array_equal(got.view(np.uint16), want.view(np.uint16))
    back = np.empty(vals.size, np.float32)
    assert l.gd_tensor_read_f32(ctx.handle, C.byref(t), back.ctypes.data, vals.size) == OK
    assert np.array_equal(back.view(np.uint32), want.astype(np.float32).view(np.uint32))
    assert l.gd_tensor_write_f32(ctx.handle, C.byref(t), vals.ctypes.data, vals.size - 1) == INVALID
    ids = _t(D, ctx, PARAMS, I32, [4])
    assert l.gd_tensor_read_f32(ctx.handle, C.byref(ids), back.ctypes.data, 4) == UNSUPPORTED
    assert l.gd_tensor_write(ctx.handle, C.byref(ids), back.ctypes.data, 12) == INVALID  # byte count mismatch
    before = t.version
    assert ctx.write(t, want) == OK and t.version == before + 1


# ---- operator front ends: status codes and success paths ---------------------------------------------------------

def test_linear_front_ends(env):
    D, l, ctx = env
    w_nk, w_kn, b = _t(D, ctx, PARAMS, F16, [16, 8]), _t(D, ctx, PARAMS, F16, [8, 16]), _t(D, ctx, PARAMS, F16, [16])
    w32 = _t(D, ctx, PARAMS, F32, [16, 8])
    out = D.GdTensor()
    x0 = _t(D, ctx, STATE, F16, [4, 8])
    assert l.gd_linear(ctx.handle, C.byref(x0), C.byref(w_kn), C.byref(b), C.byref(out)) == BAD_STATE  # output needs a step
    assert ctx.begin_step() == OK
    x = _t(D, ctx, SCRATCH, F16, [2, 3, 8])
    calls = l.gd_null_backend_op_calls()
    assert l.gd_linear(ctx.handle, C.byref(x), C.byref(w_kn), C.byref(b), C.byref(out)) == OK
    assert _last(l) == "gd_backend_linear" and l.gd_null_backend_op_calls() == calls + 1
    assert (out.rank, out.shape[0], out.shape[1], out.shape[2]) == (3, 2, 3, 16)
    assert out.storage.arena == SCRATCH and not out.is_leaf and out.dtype == F16
    assert l.gd_linear(ctx.handle, C.byref(x), C.byref(w_kn), None, C.byref(out)) == OK and _last(l) == "gd_backend_matmul"
    assert l.gd_linear_transposed_weight(ctx.handle, C.byref(x), C.byref(w_nk), C.byref(b), C.byref(out)) == OK
    assert _last(l) == "gd_backend_linear_nt" and out.shape[2] == 16
    assert l.gd_linear(ctx.handle, C.byref(x), C.byref(w_nk), None, C.byref(out)) == INVALID   # K mismatch
    assert out.storage.nbytes == 0                                                               # out is cleared first
    assert l.gd_linear(ctx.handle, C.byref(x), C.byref(w32), None, C.byref(out)) == UNSUPPORTED  # F16 only
    assert l.gd_linear(ctx.handle, C.byref(x), C.byref(w_kn), C.byref(w_kn), C.byref(out)) == INVALID  # bias rank
    assert l.gd_linear(ctx.handle, None, C.byref(w_kn), None, C.byref(out)) == INVALID
    l.gd_null_backend_fail_ops(-7)
    assert l.gd_linear(ctx.handle, C.byref(x), C.byref(w_kn), None, C.byref(out)) == -7
    assert "backend" in ctx.error()
    l.gd_null_backend_fail_ops(0)
    assert ctx.end_step() == OK


def test_swiglu_rms_norm_add_embedding_front_ends(env):
    D, l, ctx = env
    w, nw, table = _t(D, ctx, PARAMS, F16, [6, 4]), _t(D, ctx, PARAMS, F16, [12]), _t(D, ctx, PARAMS, F16, [10, 12])
    assert ctx.begin_step() == OK
    out = D.GdTensor()
    x12, odd = _t(D, ctx, SCRATCH, F16, [5, 12]), _t(D, ctx, SCRATCH, F16, [5, 7])
    assert l.gd_swiglu_split(ctx.handle, C.byref(x12), C.byref(out)) == OK and (out.shape[0], out.shape[1]) == (5, 6)
    assert l.gd_swiglu_split(ctx.handle, C.byref(odd), C.byref(out)) == INVALID
    assert l.gd_swiglu_split_linear(ctx.handle, C.byref(x12), C.byref(w), None, C.byref(out)) == OK
    assert _last(l) == "gd_backend_swiglu_split_linear" and (out.shape[0], out.shape[1]) == (5, 4)
    many = _t(D, ctx, SCRATCH, F16, [130, 12])  # many rows: gate kernel + projection, the activation span is returned
    st, mark = ctx.empty(SCRATCH, F16, [1])
    assert l.gd_swiglu_split_linear(ctx.handle, C.byref(many), C.byref(w), None, C.byref(out)) == OK
    assert _last(l) == "gd_backend_matmul" and (out.shape[0], out.shape[1]) == (130, 4)
    st, after = ctx.empty(SCRATCH, F16, [1])
    assert after.storage.offset - mark.storage.offset <= 256 + 130 * 4 * 2 + 256  # only the result stayed allocated
    assert l.gd_rms_norm(ctx.handle, C.byref(x12), C.byref(nw), 1e-5, C.byref(out)) == OK and out.shape[1] == 12
    assert l.gd_rms_norm(ctx.handle, C.byref(x12), C.byref(nw), 0.0, C.byref(out)) == INVALID
    assert l.gd_rms_norm(ctx.handle, C.byref(x12), C.byref(nw), float("nan"), C.byref(out)) == INVALID
    assert l.gd_rms_norm(ctx.handle, C.byref(odd), C.byref(nw), 1e-5, C.byref(out)) == INVALID  # weight length
    y = _t(D, ctx, SCRATCH, F16, [12])
    assert l.gd_add(ctx.handle, C.byref(x12), C.byref(y), C.byref(out)) == OK and (out.shape[0], out.shape[1]) == (5, 12)
    assert l.gd_add(ctx.handle, C.byref(x12), C.byref(odd), C.byref(out)) == INVALID and "broadcast" in ctx.error()
    ids, fids = _t(D, ctx, SCRATCH, I32, [2, 3]), _t(D, ctx, SCRATCH, F32, [3])
    assert l.gd_embedding(ctx.handle, C.byref(table), C.byref(ids), C.byref(out)) == OK
    assert (out.rank, out.shape[0], out.shape[1], out.shape[2]) == (3, 2, 3, 12)
    assert l.gd_embedding(ctx.handle, C.byref(table), C.byref(fids), C.byref(out)) != OK
    assert ctx.end_step() == OK


def test_kv_cache_append_front_ends(env):
    D, l, ctx = env
    B, T, H, Dh = 2, 6, 2, 4
    k, v = _t(D, ctx, STATE, F16, [B, T, H, Dh]), _t(D, ctx, STATE, F16, [B, T, H, Dh])
    assert ctx.begin_step() == OK
    kn, vn = _t(D, ctx, SCRATCH, F16, [B, 2, H, Dh]), _t(D, ctx, SCRATCH, F16, [B, 2, H, Dh])
    pos, cu = _t(D, ctx, SCRATCH, I32, [B]), _t(D, ctx, SCRATCH, I32, [B + 1])
    ver = k.version
    assert l.gd_kv_cache_append_at(ctx.handle, C.byref(k), C.byref(v), 4, C.byref(kn), C.byref(vn)) == OK
    assert k.version == ver + 1 and _last(l) == "gd_backend_kv_cache_append_at"
    assert l.gd_kv_cache_append_at(ctx.handle, C.byref(k), C.byref(v), 5, C.byref(kn), C.byref(vn)) == INVALID  # 2 rows do not fit
    assert l.gd_kv_cache_append_at(ctx.handle, C.byref(k), C.byref(v), -1, C.byref(kn), C.byref(vn)) == INVALID
    assert l.gd_kv_cache_append_positions(ctx.handle, C.byref(k), C.byref(v), C.byref(pos), C.byref(kn), C.byref(vn)) == OK
    fpos = _t(D, ctx, SCRATCH, F32, [B])
    assert l.gd_kv_cache_append_positions(ctx.handle, C.byref(k), C.byref(v), C.byref(fpos), C.byref(kn), C.byref(vn)) == UNSUPPORTED
    packed_k, packed_v = _t(D, ctx, SCRATCH, F16, [5, H, Dh]), _t(D, ctx, SCRATCH, F16, [5, H, Dh])
    assert l.gd_kv_cache_append_packed(ctx.handle, C.byref(k), C.byref(v), C.byref(pos), C.byref(cu), C.byref(packed_k),
                                       C.byref(packed_v)) == OK
    assert l.gd_kv_cache_append_packed(ctx.handle, C.byref(k), C.byref(v), C.byref(pos), C.byref(pos), C.byref(packed_k),
                                       C.byref(packed_v)) != OK  # cu_seqlens must have B + 1 entries
    wrong = _t(D, ctx, SCRATCH, F16, [B, 2, H, Dh + 4])
    assert l.gd_kv_cache_append_at(ctx.handle, C.byref(k), C.byref(v), 0, C.byref(wrong), C.byref(wrong)) == INVALID
    assert ctx.end_step() == OK
    assert ctx.begin_step(TRAIN) == OK  # the cache operators are inference-only
    kn = _t(D, ctx, SCRATCH, F16, [B, 1, H, Dh])
    assert l.gd_kv_cache_append_at(ctx.handle, C.byref(k), C.byref(v), 0, C.byref(kn), C.byref(kn)) == UNSUPPORTED
    assert "inference" in ctx.error()
    assert ctx.end_step() == OK


def test_attention_and_rope_front_ends(env):
    D, l, ctx = env
    B, T, H, Dh = 2, 8, 4, 128
    k, v = _t(D, ctx, STATE, F16, [B, T, 2, Dh]), _t(D, ctx, STATE, F16, [B, T, 2, Dh])
    assert ctx.begin_step() == OK
    q = _t(D, ctx, SCRATCH, F16, [B, 1, H, Dh])
    pos, scalar = _t(D, ctx, SCRATCH, I32, [B]), _t(D, ctx, SCRATCH, I32, [])
    cfg = DecodeConfig(0.0, 0, 0)
    out = D.GdTensor()
    assert l.gd_sdpa_decode_positions(ctx.handle, C.byref(q), C.byref(k), C.byref(v), C.byref(pos), C.byref(cfg), C.byref(out)) == OK
    assert (out.shape[0], out.shape[1], out.shape[2], out.shape[3]) == (B, 1, H, Dh)  # head size 128 is accepted, GQA 2:1
    assert l.gd_sdpa_decode(ctx.handle, C.byref(q), C.byref(k), C.byref(v), C.byref(scalar), C.byref(cfg), C.byref(out)) == OK
    assert l.gd_sdpa_decode(ctx.handle, C.byref(q), C.byref(k), C.byref(v), C.byref(pos), C.byref(cfg), C.byref(out)) != OK  # rank-0 tensor wanted
    assert l.gd_sdpa_decode_at(ctx.handle, C.byref(q), C.byref(k), C.byref(v), 7, C.byref(cfg), C.byref(out)) == OK
    assert l.gd_sdpa_decode_at(ctx.handle, C.byref(q), C.byref(k), C.byref(v), 8, C.byref(cfg), C.byref(out)) == INVALID  # Tq does not fit
    assert l.gd_sdpa_decode_at(ctx.handle, C.byref(q), C.byref(k), C.byref(v), -1, C.byref(cfg), C.byref(out)) == INVALID
    bad = DecodeConfig(0.0, -1, 0)
    assert l.gd_sdpa_decode_at(ctx.handle, C.byref(q), C.byref(k), C.byref(v), 0, C.byref(bad), C.byref(out)) == INVALID
    bad = DecodeConfig(float("inf"), 0, 0)
    assert l.gd_sdpa_decode_at(ctx.handle, C.byref(q), C.byref(k), C.byref(v), 0, C.byref(bad), C.byref(out)) == INVALID
    q3 = _t(D, ctx, SCRATCH, F16, [B, 1, 3, Dh])  # 3 query heads over 2 kv heads
    assert l.gd_sdpa_decode_at(ctx.handle, C.byref(q3), C.byref(k), C.byref(v), 0, C.byref(cfg), C.byref(out)) == INVALID

    N = 10
    qp, kp = _t(D, ctx, SCRATCH, F16, [N, H, Dh]), _t(D, ctx, SCRATCH, F16, [N, 2, Dh])
    cu = _t(D, ctx, SCRATCH, I32, [3])
    vc = VarlenConfig(0.0, True, 0, 0, 0)
    assert l.gd_sdpa_varlen(ctx.handle, C.byref(qp), C.byref(kp), C.byref(kp), C.byref(cu), C.byref(vc), C.byref(out)) == OK
    assert (out.rank, out.shape[0], out.shape[1], out.shape[2]) == (3, N, H, Dh)
    vc_bad = VarlenConfig(0.0, False, 0, 4, 0)  # a prefix needs the causal mask
    assert l.gd_sdpa_varlen(ctx.handle, C.byref(qp), C.byref(kp), C.byref(kp), C.byref(cu), C.byref(vc_bad), C.byref(out)) == INVALID
    one = _t(D, ctx, SCRATCH, I32, [1])
    assert l.gd_sdpa_varlen(ctx.handle, C.byref(qp), C.byref(kp), C.byref(kp), C.byref(one), C.byref(vc), C.byref(out)) == INVALID

    qkv, tok = _t(D, ctx, SCRATCH, F16, [N, 3 * H * Dh]), _t(D, ctx, SCRATCH, I32, [N])
    rope = RopeConfig(0.0, 0, False)  # theta <= 0 -> 10000, n_dims <= 0 -> head size
    oq, ok_, ov = D.GdTensor(), D.GdTensor(), D.GdTensor()
    assert l.gd_qkv_split_rope(ctx.handle, C.byref(qkv), C.byref(tok), H, Dh, C.byref(rope), C.byref(oq), C.byref(ok_), C.byref(ov)) == OK
    assert (oq.shape[0], oq.shape[1], oq.shape[2]) == (N, H, Dh) and (ov.shape[1], ov.shape[2]) == (H, Dh)
    partial = RopeConfig(10000.0, Dh // 2, False)
    assert l.gd_qkv_split_rope(ctx.handle, C.byref(qkv), C.byref(tok), H, Dh, C.byref(partial), C.byref(oq), C.byref(ok_), C.byref(ov)) == UNSUPPORTED
    odd = RopeConfig(10000.0, 3, False)
    assert l.gd_qkv_split_rope(ctx.handle, C.byref(qkv), C.byref(tok), H, Dh, C.byref(odd), C.byref(oq), C.byref(ok_), C.byref(ov)) == INVALID
    assert l.gd_qkv_split_rope(ctx.handle, C.byref(qkv), C.byref(tok), H + 1, Dh, C.byref(rope), C.byref(oq), C.byref(ok_), C.byref(ov)) == INVALID
    assert ctx.end_step() == OK


# ---- decoder: weights follow the reference's seeded initialisation, on the CPU ----------------------------------

def test_decoder_weights_equal_the_oracle_without_a_gpu(host, oracle):
    pkg, D = host
    cfg = D.gpt_config(96, 32, 2, 4, 8, 48, 16, 2, 0, False, 1000)
    dev = D.GptDecoder(cfg, max_prefill_tokens=8)
    ref = oracle.Decoder(96, 32, 2, 4, 8, 48, 16, 2, 0, 1000, False)
    try:
        for name in ("embed", "lm_head", "final_norm", "lm_bias"):
            assert np.array_equal(dev.read_tensor(name).view(np.uint16), ref.tensor(name).view(np.uint16)), name
        for layer in (0, 1):
            for name in ("attn_norm", "w_qkv", "b_qkv", "w_attn", "w_upgate", "w_down", "b_down"):
                assert np.array_equal(dev.read_tensor(name, layer).view(np.uint16),
                                      ref.tensor(name, layer).view(np.uint16)), (name, layer)
        assert not dev.read_tensor("k_cache", 1).any()
    finally:
        dev.close()
        ref.close()


# ---- decoder: the accounting of a resident session, on the CPU ----------------------------------------------------

def test_resident_sessions_count_steps_and_refuse_what_does_not_fit(host):
    """The device-less backend records graphs that hold nothing and counts their replays, so the tokens mean
    nothing here; what is held is the order of calls a session accepts, how many steps it lets run, and what the
    decoder refuses while one is open."""
    pkg, D = host
    l = D.lib()
    l.gd_null_backend_graph_launches.restype = C.c_uint64
    cfg = D.gpt_config(96, 32, 2, 4, 8, 48, 32, 3, 0, True, 1000)
    dev = D.GptDecoder(cfg, max_prefill_tokens=24)
    ids, cu = np.arange(20, dtype=np.int32), np.array([0, 8, 9, 20], np.int32)
    try:
        with pytest.raises(pkg.GdError) as e:  # no session open
            dev.resident_run(1)
        assert e.value.status == BAD_STATE
        dev.prefill(ids, cu)
        before = l.gd_null_backend_graph_launches()
        dev.resident_begin([1, 2, 3], 5)  # the first step runs inside begin
        dev.resident_run(3)
        assert l.gd_null_backend_graph_launches() == before + 3
        with pytest.raises(pkg.GdError) as e:  # 1 + 3 + 2 > 5
            dev.resident_run(2)
        assert e.value.status == INVALID
        for call in (lambda: dev.prefill(ids, cu), lambda: dev.step([1, 2, 3]), lambda: dev.generate(ids, cu, 4),
                     lambda: dev.resident_begin([1, 2, 3], 2), lambda: dev.load_checkpoint("/nonexistent", True)):
            with pytest.raises(pkg.GdError) as e:
                call()
            assert e.value.status == -4, "busy while a session is open"
        dev.resident_run(1)
        out, gaps = dev.resident_end()
        assert out.shape == (5, 3)
        assert list(dev.positions) == [8 + 5, 1 + 5, 11 + 5]
        # a sampled session starts from the prefill's logits: its first pick costs no step
        dev.prefill(ids, cu)
        before = l.gd_null_backend_graph_launches()
        dev.resident_begin_sampled(ids, cu, 6, 0.8, min_p=0.05, repetition_penalty=1.1, stop_token=5)
        dev.resident_run(4)
        assert l.gd_null_backend_graph_launches() == before + 4
        with pytest.raises(pkg.GdError):
            dev.resident_run(1)
        out, _ = dev.resident_end()
        assert out.shape == (6, 3)
        # rows stop where the context ends: 32 - 11 = 21 tokens fit the longest row, whatever max_new asks
        rows = dev.generate(ids, cu, 100, temperature=0.0)
        assert [len(r) <= 32 - n for r, n in zip(rows, (8, 1, 11))] == [True] * 3
        with pytest.raises(pkg.GdError) as e:  # empty prompt
            dev.generate(ids, np.array([0, 0, 9, 20], np.int32), 4)
        assert e.value.status == INVALID
    finally:
        dev.close()
