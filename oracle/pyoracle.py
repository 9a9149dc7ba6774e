"""ctypes front-end of the host oracle (oracle/nvtext_oracle.cpp).

TEST INFRASTRUCTURE: imported only by tests/, by ``__graft_entry__.smoke`` and
by the ``cpu_baseline`` leg of bench.py, always as the checker.  The product
package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# NVTEXT_ORACLE_LIB names another build of the same source (the sanitizer build of `make SAN=1`)
_LIB_PATH = os.environ.get("NVTEXT_ORACLE_LIB") or os.path.join(_HERE, "libnvtext_oracle.so")
_lib = None

OK, INVALID_ARGUMENT, OVERFLOW_ERROR, LOGIC_ERROR = 0, 1, 2, 3


class OracleError(Exception):
    def __init__(self, code: int):
        super().__init__({1: "invalid_argument", 2: "overflow_error", 3: "logic_error"}.get(code, str(code)))
        self.code = code


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "nvtext_oracle.cpp")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.oracle_murmur3_x86_32.restype = C.c_uint32
        L.oracle_murmur3_x86_32.argtypes = [C.c_void_p, C.c_int64, C.c_uint32]
        L.oracle_murmur3_x64_128.restype = None
        L.oracle_murmur3_x64_128.argtypes = [C.c_void_p, C.c_int64, C.c_uint64, C.c_void_p]
        col = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int32, C.c_int32, C.c_int32]
        L.oracle_minhash.restype = C.c_int
        L.oracle_minhash.argtypes = col + [C.c_uint32, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int,
                                           C.c_void_p, C.c_void_p, C.POINTER(C.c_int64)]
        L.oracle_minhash64.restype = C.c_int
        L.oracle_minhash64.argtypes = col + [C.c_uint64, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int,
                                             C.c_void_p, C.c_void_p, C.POINTER(C.c_int64)]
        lcol = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int32, C.c_int32]
        L.oracle_minhash_ngrams.restype = C.c_int
        L.oracle_minhash_ngrams.argtypes = lcol + [C.c_int32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_int32, C.c_int,
                                                   C.c_void_p, C.c_void_p, C.POINTER(C.c_int64)]
        L.oracle_minhash64_ngrams.restype = C.c_int
        L.oracle_minhash64_ngrams.argtypes = lcol + [C.c_int32, C.c_uint64, C.c_void_p, C.c_void_p, C.c_int32, C.c_int,
                                                     C.c_void_p, C.c_void_p, C.POINTER(C.c_int64)]
        L.oracle_jaccard_index.restype = C.c_int
        L.oracle_jaccard_index.argtypes = col + col + [C.c_int32, C.c_int, C.c_void_p, C.c_void_p, C.POINTER(C.c_int32),
                                                       C.POINTER(C.c_int32)]
        L.oracle_vocab_create.restype = C.c_int
        L.oracle_vocab_create.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int32, C.c_int32, C.c_int32,
                                          C.POINTER(C.c_void_p)]
        L.oracle_vocab_destroy.restype = None
        L.oracle_vocab_destroy.argtypes = [C.c_void_p]
        L.oracle_vocab_unk_id.restype = C.c_int32
        L.oracle_vocab_unk_id.argtypes = [C.c_void_p]
        L.oracle_wordpiece_tokenize.restype = C.c_int
        L.oracle_wordpiece_tokenize.argtypes = [C.c_void_p] + col + [
            C.c_int32, C.c_int, C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int64), C.POINTER(C.c_int32)]
        L.oracle_normalize_characters.restype = C.c_int
        L.oracle_normalize_characters.argtypes = col + [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int32,
                                                        C.c_int, C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int64)]
        L.oracle_free.restype = None
        L.oracle_free.argtypes = [C.c_void_p]
        L.oracle_copy_bitmask.restype = None
        L.oracle_copy_bitmask.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]
        L.oracle_hardware_threads.restype = C.c_int
        _lib = L
    return _lib


def _p(a: Optional[np.ndarray]):
    if a is None:
        return None
    return a.ctypes.data_as(C.c_void_p)


def _col_args(col):
    chars = np.ascontiguousarray(col.chars, dtype=np.uint8)
    offsets = np.ascontiguousarray(col.offsets)
    assert offsets.dtype in (np.int32, np.int64)
    mask = None if col.mask is None else np.ascontiguousarray(col.mask, dtype=np.uint32)
    keep = (chars, offsets, mask)
    return keep, [_p(chars) if chars.size else None, _p(offsets) if offsets.size else None,
                  int(offsets.dtype == np.int64), _p(mask), int(col.size), int(col.offset), int(col.null_count)]


def murmur3_x86_32(data: bytes, seed: int = 0) -> int:
    buf = np.frombuffer(data, dtype=np.uint8)
    return int(lib().oracle_murmur3_x86_32(_p(buf) if buf.size else None, len(data), seed))


def murmur3_x64_128(data: bytes, seed: int = 0):
    buf = np.frombuffer(data, dtype=np.uint8)
    out = np.zeros(2, dtype=np.uint64)
    lib().oracle_murmur3_x64_128(_p(buf) if buf.size else None, len(data), seed, _p(out))
    return int(out[0]), int(out[1])


def hardware_threads() -> int:
    return int(lib().oracle_hardware_threads())


def copy_bitmask(col) -> Optional[np.ndarray]:
    if col.mask is None:
        return None
    out = np.zeros((col.size + 31) // 32, dtype=np.uint32)
    if col.size:
        m = np.ascontiguousarray(col.mask, dtype=np.uint32)
        lib().oracle_copy_bitmask(_p(m), col.offset, col.size, _p(out))
    return out


def _minhash(col, seed, a, b, width, dtype, fn, nthreads):
    from cudf_amd.arrow_host import HostListColumn  # plain numpy container
    a = np.ascontiguousarray(a, dtype=dtype)
    b = np.ascontiguousarray(b, dtype=dtype)
    if a.size != b.size:
        raise OracleError(INVALID_ARGUMENT)
    keep, cargs = _col_args(col)
    P = int(a.size)
    rows = int(col.size)
    ok_size = width >= 2 and P > 0 and rows * P < 2**31 - 1
    offsets = np.zeros(rows + 1, dtype=np.int32)
    child = np.zeros(rows * P if ok_size else 0, dtype=dtype)
    n = C.c_int64(0)
    rc = fn(*cargs, seed, _p(a) if P else None, _p(b) if P else None, P, width, nthreads,
            _p(offsets), _p(child) if child.size else None, C.byref(n))
    if rc != OK:
        raise OracleError(rc)
    return HostListColumn(offsets, child[:n.value].copy(), copy_bitmask(col), rows, int(col.null_count))


def minhash(col, seed, a, b, width, nthreads: int = 1):
    return _minhash(col, seed, a, b, width, np.uint32, lib().oracle_minhash, nthreads)


def minhash64(col, seed, a, b, width, nthreads: int = 1):
    return _minhash(col, seed, a, b, width, np.uint64, lib().oracle_minhash64, nthreads)


def _minhash_ngrams(col, ngrams, seed, a, b, dtype, fn, nthreads):
    """col: cudf_amd.arrow_host.HostListStringsColumn."""
    from cudf_amd.arrow_host import HostListColumn
    a = np.ascontiguousarray(a, dtype=dtype)
    b = np.ascontiguousarray(b, dtype=dtype)
    if a.size != b.size:
        raise OracleError(INVALID_ARGUMENT)
    loffs = np.ascontiguousarray(col.offsets, dtype=np.int32)
    lmask = None if col.mask is None else np.ascontiguousarray(col.mask, dtype=np.uint32)
    keep, cargs = _col_args(col.child)
    P = int(a.size)
    rows = int(col.size)
    ok_size = ngrams >= 2 and P > 0 and rows * P < 2**31 - 1
    offsets = np.zeros(rows + 1, dtype=np.int32)
    child = np.zeros(rows * P if ok_size else 0, dtype=dtype)
    n = C.c_int64(0)
    rc = fn(_p(loffs) if loffs.size else None, _p(lmask), rows, int(col.offset), int(col.null_count), *cargs[:6],
            ngrams, seed, _p(a) if P else None, _p(b) if P else None, P, nthreads,
            _p(offsets), _p(child) if child.size else None, C.byref(n))
    if rc != OK:
        raise OracleError(rc)
    return HostListColumn(offsets, child[:n.value].copy(), copy_bitmask(col), rows, int(col.null_count))


def minhash_ngrams(col, ngrams, seed, a, b, nthreads: int = 1):
    return _minhash_ngrams(col, ngrams, seed, a, b, np.uint32, lib().oracle_minhash_ngrams, nthreads)


def minhash64_ngrams(col, ngrams, seed, a, b, nthreads: int = 1):
    return _minhash_ngrams(col, ngrams, seed, a, b, np.uint64, lib().oracle_minhash64_ngrams, nthreads)


def jaccard_index(col1, col2, width, nthreads: int = 1):
    from cudf_amd.arrow_host import HostFixedColumn
    keep1, a1 = _col_args(col1)
    keep2, a2 = _col_args(col2)
    rows = int(col1.size)
    out = np.zeros(rows, dtype=np.float32)
    mask = np.zeros((rows + 31) // 32, dtype=np.uint32)
    nulls = C.c_int32(0)
    has_mask = C.c_int32(0)
    rc = lib().oracle_jaccard_index(*a1, *a2, width, nthreads, _p(out) if rows else None, _p(mask) if rows else None,
                                    C.byref(nulls), C.byref(has_mask))
    if rc != OK:
        raise OracleError(rc)
    return HostFixedColumn(out, mask if has_mask.value and rows else None, rows, int(nulls.value))


class Vocabulary:
    def __init__(self, col):
        keep, cargs = _col_args(col)
        h = C.c_void_p()
        rc = lib().oracle_vocab_create(cargs[0], cargs[1], cargs[2], cargs[4], cargs[5], cargs[6], C.byref(h))
        if rc != OK:
            raise OracleError(rc)
        self._h = h
        self.unk_id = int(lib().oracle_vocab_unk_id(h))

    def __del__(self):
        # at interpreter exit the module's globals may be gone already: then the process ends with the memory anyway
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            try:
                _lib.oracle_vocab_destroy(h)
            except Exception:
                pass


def wordpiece_tokenize(col, vocab: Vocabulary, max_words_per_row: int = 0, nthreads: int = 1):
    from cudf_amd.arrow_host import HostListColumn
    keep, cargs = _col_args(col)
    rows = int(col.size)
    offsets = np.zeros(rows + 1, dtype=np.int32)
    toks = C.c_void_p()
    n = C.c_int64(0)
    kind = C.c_int32(0)
    rc = lib().oracle_wordpiece_tokenize(vocab._h, *cargs, max_words_per_row, nthreads, _p(offsets),
                                         C.byref(toks), C.byref(n), C.byref(kind))
    if rc != OK:
        raise OracleError(rc)
    if kind.value == 2:   # canonical empty list column: 0 rows, 0-length offsets
        return HostListColumn(np.zeros(0, np.int32), np.zeros(0, np.int32), None, 0, 0)
    if kind.value == 1:   # all rows null
        return HostListColumn(offsets, np.zeros(0, np.int32), np.zeros((rows + 31) // 32, np.uint32), rows, rows)
    child = np.ctypeslib.as_array(C.cast(toks, C.POINTER(C.c_int32)), shape=(max(n.value, 1),))[:n.value].copy()
    lib().oracle_free(toks)
    return HostListColumn(offsets, child, copy_bitmask(col), rows, int(col.null_count))
