"""Seeded synthetic workloads: the five benchmark/parity configurations.

Thin ctypes front-end of datagen.cpp.  Every workload is a pure function of its seed
and `scale` (the row count multiplier), independent of the thread count.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass
from typing import Optional

import numpy as np

from ..arrow_host import HostListStringsColumn, HostStringsColumn

_HERE = os.path.dirname(os.path.abspath(__file__))
# NVTEXT_DATAGEN_LIB names another build of the same source (the sanitizer build of `make SAN=1`)
_LIB_PATH = os.environ.get("NVTEXT_DATAGEN_LIB") or os.path.join(_HERE, "libnvtext_datagen.so")
_lib = None


class _RowsConfig(C.Structure):
    _fields_ = [
        ("rows", C.c_int64), ("seed", C.c_uint64), ("mean_bytes", C.c_double), ("sigma", C.c_double),
        ("cap_bytes", C.c_int64), ("min_bytes", C.c_int64), ("zipf_s", C.c_double), ("p_oov", C.c_double),
        ("p_null", C.c_double), ("p_empty", C.c_double), ("words_lo", C.c_int32), ("words_hi", C.c_int32),
        ("oov_lo", C.c_int32), ("oov_hi", C.c_int32), ("multilingual", C.c_int32), ("uniform_words", C.c_int32),
    ]


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "datagen.cpp")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.datagen_vocab_create.restype = C.c_void_p
        L.datagen_vocab_create.argtypes = [C.c_int, C.c_int64, C.c_uint64, C.POINTER(C.c_int64)]
        L.datagen_vocab_finish.restype = None
        L.datagen_vocab_finish.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.datagen_rows_begin.restype = C.c_void_p
        L.datagen_rows_begin.argtypes = [C.POINTER(_RowsConfig), C.c_void_p, C.c_void_p, C.c_int64, C.c_int,
                                         C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        L.datagen_rows_finish.restype = None
        L.datagen_rows_finish.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _threads() -> int:
    return max(1, min(16, os.cpu_count() or 1))


VOCAB_BERT, VOCAB_LEXICON, VOCAB_MULTILINGUAL = 0, 1, 2


def make_vocab(kind: int, size: int, seed: int) -> HostStringsColumn:
    L = _load()
    n = C.c_int64(0)
    h = L.datagen_vocab_create(kind, size, seed, C.byref(n))
    chars = np.empty(max(n.value, 1), np.uint8)[: n.value]
    offsets = np.empty(size + 1, np.int64)
    L.datagen_vocab_finish(h, chars.ctypes.data_as(C.c_void_p) if n.value else None, offsets.ctypes.data_as(C.c_void_p))
    return HostStringsColumn(chars, offsets.astype(np.int32), None, size, 0, 0)


def make_rows(lexicon: Optional[HostStringsColumn], *, rows: int, seed: int, mean_bytes: float = 256.0, sigma: float = 0.6,
              cap_bytes: int = 1 << 40, min_bytes: int = 1, zipf_s: float = 1.1, p_oov: float = 0.0, p_null: float = 0.0,
              p_empty: float = 0.0, words_lo: int = 0, words_hi: int = 0, oov_lo: int = 3, oov_hi: int = 10,
              multilingual: bool = False, uniform_words: bool = False, offsets_dtype=np.int32) -> HostStringsColumn:
    L = _load()
    cfg = _RowsConfig(rows, seed, mean_bytes, sigma, cap_bytes, min_bytes, zipf_s, p_oov, p_null, p_empty, words_lo, words_hi,
                      oov_lo, oov_hi, int(multilingual), int(uniform_words))
    total, nulls = C.c_int64(0), C.c_int64(0)
    if lexicon is not None:
        lc = np.ascontiguousarray(lexicon.chars)
        lo = np.ascontiguousarray(lexicon.offsets, dtype=np.int64)
        h = L.datagen_rows_begin(C.byref(cfg), lc.ctypes.data_as(C.c_void_p), lo.ctypes.data_as(C.c_void_p), lexicon.size,
                                 _threads(), C.byref(total), C.byref(nulls))
    else:
        h = L.datagen_rows_begin(C.byref(cfg), None, None, 0, _threads(), C.byref(total), C.byref(nulls))
    chars = np.empty(max(total.value, 1), np.uint8)[: total.value]
    offsets = np.empty(rows + 1, np.int64)
    mask = np.empty((rows + 31) // 32, np.uint32) if nulls.value else None
    L.datagen_rows_finish(h, chars.ctypes.data_as(C.c_void_p) if total.value else None, offsets.ctypes.data_as(C.c_void_p),
                          mask.ctypes.data_as(C.c_void_p) if mask is not None else None)
    if offsets_dtype == np.int32:
        if total.value >= 2**31:
            raise OverflowError("chars do not fit int32 offsets")
        offsets = offsets.astype(np.int32)
    return HostStringsColumn(chars, offsets, mask, rows, 0, int(nulls.value))


@dataclass
class Workload:
    name: str
    rows: HostStringsColumn
    vocab: Optional[HostStringsColumn]
    params: dict


def config1(scale: float = 1.0) -> Workload:
    """Host-oracle smoke: 10k ASCII rows of 5-40 uniform 1-12 letter words, 2 % null, 30,522-entry vocabulary;
    tokenize max_words_per_row=0, then minhash uint32 width 4 seed 0 with 64 (a, b) pairs."""
    vocab = make_vocab(VOCAB_BERT, 30522, seed=1001)
    rows = make_rows(None, rows=int(10000 * scale), seed=1, words_lo=5, words_hi=40, p_null=0.02, uniform_words=True)
    return Workload("C1", rows, vocab, dict(max_words_per_row=0, width=4, seed=0, P=64, hash_bits=32, param_seed=11))


def config2(scale: float = 1.0) -> Workload:
    """wordpiece_tokenize throughput: 4M rows, lognormal mean 256 B sigma 0.6 cap 4 KB, Zipf(1.1) over the vocabulary's
    stems, 15 % out-of-vocabulary random strings, int32 offsets, max_words_per_row=128."""
    vocab = make_vocab(VOCAB_BERT, 30522, seed=1001)
    rows = make_rows(vocab, rows=int(4_000_000 * scale), seed=2, mean_bytes=256.0, sigma=0.6, cap_bytes=4096, zipf_s=1.1,
                     p_oov=0.15, min_bytes=2)
    return Workload("C2", rows, vocab, dict(max_words_per_row=128))


def config3(scale: float = 1.0) -> Workload:
    """minhash uint32 throughput: 2M docs, lognormal mean 2 KB sigma 0.8, 50k-word Zipf lexicon;
    width 5, seed 42, 256 (a, b) pairs."""
    lex = make_vocab(VOCAB_LEXICON, 50000, seed=1003)
    rows = make_rows(lex, rows=int(2_000_000 * scale), seed=3, mean_bytes=2048.0, sigma=0.8, zipf_s=1.1, min_bytes=2,
                     offsets_dtype=np.int64 if scale > 0.45 else np.int32)
    return Workload("C3", rows, None, dict(width=5, seed=42, P=256, hash_bits=32, param_seed=33))


def config4(scale: float = 1.0) -> Workload:
    """minhash64 long documents: 100k docs, lognormal mean 16 KB capped at 1 MB (sigma 1.5 so that rows above 256 KiB
    occur), 10 % null, 1 % empty; width 5, seed 7, 128 (a, b) pairs."""
    lex = make_vocab(VOCAB_LEXICON, 50000, seed=1003)
    rows = make_rows(lex, rows=int(100_000 * scale), seed=4, mean_bytes=16384.0, sigma=1.5, cap_bytes=1 << 20, zipf_s=1.1,
                     p_null=0.10, p_empty=0.01, min_bytes=2)
    return Workload("C4", rows, None, dict(width=5, seed=7, P=128, hash_bits=64, param_seed=44))


def config5(scale: float = 1.0) -> Workload:
    """UTF-8 pipeline: 8M rows, mean 512 B, int64 offsets, per-word script mix 70 % ASCII / 20 % Latin-1 / 10 % CJK with
    punctuation words, 250k-entry multilingual vocabulary; tokenize max_words_per_row=256, then minhash64 width 8, 64 pairs."""
    vocab = make_vocab(VOCAB_MULTILINGUAL, 250000, seed=1005)
    rows = make_rows(vocab, rows=int(8_000_000 * scale), seed=5, mean_bytes=512.0, sigma=0.6, cap_bytes=8192, zipf_s=1.1,
                     p_oov=0.10, multilingual=True, min_bytes=2, offsets_dtype=np.int64)
    return Workload("C5", rows, vocab, dict(max_words_per_row=256, width=8, seed=5, P=64, hash_bits=64, param_seed=55))


def words_as_lists(rows: HostStringsColumn) -> HostListStringsColumn:
    """The rows of a generated strings column (single spaces, none leading or trailing) as LIST<STRING> rows over the
    same chars: element = a word together with the space that follows it, so that the elements of a row tile its bytes
    (the layout a tokenizer's output has when it keeps the separators).  Null rows stay null, empty rows are empty lists."""
    chars = np.ascontiguousarray(rows.chars)
    roff = np.ascontiguousarray(rows.offsets).astype(np.int64)
    assert rows.offset == 0
    after_space = np.flatnonzero(chars == 0x20).astype(np.int64) + 1
    starts = np.union1d(after_space, roff[:-1][np.diff(roff) > 0])
    child_offsets = np.concatenate([starts, roff[-1:]]).astype(rows.offsets.dtype)
    list_offsets = np.searchsorted(starts, roff, side="left").astype(np.int32)
    child = HostStringsColumn(chars, child_offsets, None, int(starts.size), 0, 0)
    return HostListStringsColumn(list_offsets, child, rows.mask, rows.size, 0, rows.null_count)


CONFIGS = {"C1": config1, "C2": config2, "C3": config3, "C4": config4, "C5": config5}


def make_params(P: int, bits: int, seed: int):
    """Seeded (a, b) permutation parameters; a is never 0."""
    rng = np.random.default_rng(seed)
    if bits == 32:
        a = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
        b = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
    else:
        a = rng.integers(1, 2**64, P, dtype=np.uint64)
        b = rng.integers(0, 2**64, P, dtype=np.uint64)
    return a, b
