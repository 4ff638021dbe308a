"""ctypes binding of the byte-level BPE tokenizer (gd_tokenizer.h)."""
import ctypes as C
import os

import numpy as np

from . import GD_OK, GdError, lib as _base_lib

_vp = C.c_void_p
_declared = False


class TokenizerConfig(C.Structure):  # gd_tokenizer_config
    _fields_ = [("split_digits", C.c_int), ("allow_special", C.c_int)]


def lib():
    global _declared
    l = _base_lib()
    if not _declared:
        l.gd_bpe_tokenizer_load.argtypes = [C.c_char_p, C.POINTER(TokenizerConfig), C.POINTER(_vp)]
        l.gd_tokenizer_destroy.argtypes = [_vp]
        l.gd_tokenizer_destroy.restype = None
        l.gd_tokenizer_encode.argtypes = [_vp, C.c_char_p, C.POINTER(C.POINTER(C.c_int32)), C.POINTER(C.c_int)]
        l.gd_tokenizer_decode.argtypes = [_vp, _vp, C.c_int, C.POINTER(_vp)]
        l.gd_tokenizer_id.argtypes = [_vp, C.c_char_p, C.POINTER(C.c_int32)]
        l.gd_tokenizer_vocab_size.argtypes = [_vp]
        l.gd_tokenizer_hash.argtypes = [_vp]
        l.gd_tokenizer_hash.restype = C.c_uint64
        l.gd_tokenizer_free.argtypes = [_vp]
        l.gd_tokenizer_free.restype = None
        _declared = True
    return l


class Tokenizer:
    """A vocabulary file written by the reference's gd_bpe_tokenizer_save.  split_digits / allow_special None: as the
    file says / specials allowed (a NULL configuration)."""

    def __init__(self, path, split_digits=None, allow_special=None):
        self.handle = _vp()
        cfg = None
        if split_digits is not None or allow_special is not None:
            cfg = C.byref(TokenizerConfig(1 if split_digits is None else int(split_digits),
                                          1 if allow_special is None else int(allow_special)))
        st = lib().gd_bpe_tokenizer_load(os.fsencode(path), cfg, C.byref(self.handle))
        if st != GD_OK:
            self.handle = None
            raise GdError(st, f"gd_bpe_tokenizer_load({path})")

    def close(self):
        if getattr(self, "handle", None):
            lib().gd_tokenizer_destroy(self.handle)
            self.handle = None

    __del__ = close

    def encode(self, text):
        """text: str (encoded as UTF-8) or bytes without NUL.  Returns an int32 array."""
        raw = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        ids, n = C.POINTER(C.c_int32)(), C.c_int()
        st = lib().gd_tokenizer_encode(self.handle, raw, C.byref(ids), C.byref(n))
        if st != GD_OK:
            raise GdError(st, "gd_tokenizer_encode")
        try:
            return np.ctypeslib.as_array(ids, shape=(n.value,)).astype(np.int32) if n.value else np.zeros(0, np.int32)
        finally:
            lib().gd_tokenizer_free(ids)

    def decode(self, ids):
        """ids to bytes (the tokens' bytes, not necessarily valid UTF-8)."""
        ids = np.ascontiguousarray(ids, np.int32)
        out = _vp()
        st = lib().gd_tokenizer_decode(self.handle, ids.ctypes.data_as(_vp), ids.size, C.byref(out))
        if st != GD_OK:
            raise GdError(st, "gd_tokenizer_decode")
        try:
            return C.string_at(out)
        finally:
            lib().gd_tokenizer_free(out)

    def token_id(self, special):
        out = C.c_int32()
        st = lib().gd_tokenizer_id(self.handle, special.encode(), C.byref(out))
        if st != GD_OK:
            raise GdError(st, f"gd_tokenizer_id({special})")
        return out.value

    @property
    def vocab_size(self):
        return lib().gd_tokenizer_vocab_size(self.handle)

    @property
    def hash(self):
        return lib().gd_tokenizer_hash(self.handle)
