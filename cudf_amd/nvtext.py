"""Python host side of the nvtext hot path, over the C ABI.

Mirrors the call contract of pylibcudf's bindings for this path
(python/pylibcudf/pylibcudf/nvtext/minhash.pyx:33-141,
 python/pylibcudf/pylibcudf/nvtext/wordpiece_tokenize.pyx:22-97): same function names,
argument order and error behaviour (std::invalid_argument -> ValueError,
std::overflow_error -> OverflowError, as libcudf_exception_handler maps them).

PyTorch is used only as the owner of device memory and the provider of the HIP stream;
every computation happens in libnvtext_amd.so.
"""
from __future__ import annotations

import ctypes as C
import sys
from dataclasses import dataclass
from typing import Dict, Optional

import numpy as np

from . import _capi
from .arrow_host import HostFixedColumn, HostListColumn, HostStringsColumn


def _torch():
    import torch
    return torch


class _TorchAllocator:
    """nvtext_amd_allocator backed by torch's caching allocator (stream-ordered on the
    current stream).  Buffers handed back in a result stay alive in `take()`n tensors."""

    def __init__(self):
        self.live: Dict[int, object] = {}
        # for tests of the library's error paths: when set to n, the n + 1-th request from now and all later ones
        # are refused until it is set to None again
        self.fail_after: Optional[int] = None
        torch = _torch()

        def _alloc(ctx, nbytes, stream):
            if self.fail_after is not None:
                if self.fail_after == 0:
                    return None
                self.fail_after -= 1
            try:
                t = torch.empty(int(nbytes), dtype=torch.uint8, device="cuda")
            except Exception:  # out of memory -> NULL, reported as ALLOC_FAILED
                return None
            self.live[t.data_ptr()] = t
            return t.data_ptr()

        def _free(ctx, ptr, nbytes, stream):
            self.live.pop(int(ptr) if ptr else 0, None)

        self._alloc_cb = _capi.ALLOC_FN(_alloc)
        self._free_cb = _capi.DEALLOC_FN(_free)
        self.struct = _capi.Allocator(None, self._alloc_cb, self._free_cb)

    def take(self, ptr):
        return self.live.pop(int(ptr), None) if ptr else None


_allocator: Optional[_TorchAllocator] = None


def _mr() -> _TorchAllocator:
    global _allocator
    if _allocator is None:
        _allocator = _TorchAllocator()
    return _allocator


def _stream_handle() -> int:
    return int(_torch().cuda.current_stream().cuda_stream)


def _raise(status: int):
    msg = _capi.load().nvtext_amd_last_error().decode("utf-8", "replace")
    if status == _capi.INVALID_ARGUMENT:
        raise ValueError(msg)
    if status == _capi.OVERFLOW:
        raise OverflowError(msg)
    if status == _capi.ALLOC_FAILED:
        raise MemoryError(msg)
    raise RuntimeError(msg)


@dataclass
class DeviceStringsColumn:
    """Arrow-layout strings column in HBM (torch tensors own the buffers)."""
    chars: object            # uint8 tensor
    offsets: object          # int32 / int64 tensor (parent_size + 1 entries) or None
    mask: object             # int32 tensor holding the uint32 validity words, or None
    size: int
    offset: int = 0
    null_count: int = 0

    @staticmethod
    def from_host(h: HostStringsColumn, device: str = "cuda") -> "DeviceStringsColumn":
        torch = _torch()
        chars = torch.from_numpy(np.ascontiguousarray(h.chars)).to(device)
        offsets = torch.from_numpy(np.ascontiguousarray(h.offsets)).to(device) if h.offsets.size else None
        mask = None
        if h.mask is not None:
            mask = torch.from_numpy(np.ascontiguousarray(h.mask).view(np.int32)).to(device)
        return DeviceStringsColumn(chars, offsets, mask, int(h.size), int(h.offset), int(h.null_count))

    def slice(self, lo: int, hi: int, null_count: int) -> "DeviceStringsColumn":
        return DeviceStringsColumn(self.chars, self.offsets, self.mask, hi - lo, self.offset + lo, null_count)

    def to_host(self) -> HostStringsColumn:
        torch = _torch()
        torch.cuda.current_stream().synchronize()
        offsets = self.offsets.cpu().numpy().copy() if self.offsets is not None else np.zeros(0, np.int32)
        mask = self.mask.cpu().numpy().view(np.uint32).copy() if self.mask is not None else None
        return HostStringsColumn(self.chars.cpu().numpy().copy(), offsets, mask, self.size, self.offset, self.null_count)

    def _c(self) -> _capi.StringsColumn:
        torch = _torch()
        is64 = 0
        if self.offsets is not None:
            if self.offsets.dtype == torch.int64:
                is64 = 1
            elif self.offsets.dtype != torch.int32:
                raise TypeError("offsets must be int32 or int64")
        return _capi.StringsColumn(
            self.chars.data_ptr() if self.chars is not None and self.chars.numel() else None,
            self.offsets.data_ptr() if self.offsets is not None else None,
            is64,
            self.mask.data_ptr() if self.mask is not None else None,
            self.size, self.offset, self.null_count)


@dataclass
class DeviceListStringsColumn:
    """LIST<STRING> column in HBM: int32 list offsets, optional row validity, a strings child."""
    offsets: object          # int32 tensor (parent_size + 1 entries) or None for an empty column
    child: DeviceStringsColumn
    mask: object
    size: int
    offset: int = 0
    null_count: int = 0

    @staticmethod
    def from_host(h, device: str = "cuda") -> "DeviceListStringsColumn":
        torch = _torch()
        offsets = torch.from_numpy(np.ascontiguousarray(h.offsets, dtype=np.int32)).to(device) if h.offsets.size else None
        mask = None
        if h.mask is not None:
            mask = torch.from_numpy(np.ascontiguousarray(h.mask).view(np.int32)).to(device)
        return DeviceListStringsColumn(offsets, DeviceStringsColumn.from_host(h.child, device), mask, int(h.size), int(h.offset),
                                       int(h.null_count))

    def slice(self, lo: int, hi: int, null_count: int) -> "DeviceListStringsColumn":
        return DeviceListStringsColumn(self.offsets, self.child, self.mask, hi - lo, self.offset + lo, null_count)

    def _c(self) -> _capi.ListStringsColumn:
        torch = _torch()
        if self.offsets is not None and self.offsets.dtype != torch.int32:
            raise TypeError("list offsets must be int32")
        return _capi.ListStringsColumn(
            self.offsets.data_ptr() if self.offsets is not None else None,
            self.mask.data_ptr() if self.mask is not None else None,
            self.size, self.offset, self.null_count, self.child._c())


@dataclass
class DeviceListColumn:
    """LIST result in HBM.  offsets: int32 tensor; child: raw tensor viewed as child_dtype."""
    offsets: object
    child: object
    mask: object
    size: int
    null_count: int
    child_dtype: np.dtype
    child_size: int

    def to_host(self) -> HostListColumn:
        torch = _torch()
        torch.cuda.current_stream().synchronize()
        offsets = (self.offsets.cpu().numpy().view(np.int32)[: self.size + 1].copy()
                   if self.offsets is not None else np.zeros(0, np.int32))
        if self.child is not None:
            child = self.child.cpu().numpy().view(self.child_dtype)[: self.child_size].copy()
        else:
            child = np.zeros(0, self.child_dtype)
        mask = None
        if self.mask is not None:
            mask = self.mask.cpu().numpy().view(np.uint32)[: (self.size + 31) // 32].copy()
        return HostListColumn(offsets, child, mask, self.size, self.null_count)


@dataclass
class DeviceFixedColumn:
    """Fixed-width result in HBM (FLOAT32 here): raw data tensor, optional validity words."""
    data: object
    mask: object
    size: int
    null_count: int
    dtype: np.dtype

    def to_host(self) -> "HostFixedColumn":
        torch = _torch()
        torch.cuda.current_stream().synchronize()
        values = (self.data.cpu().numpy().view(self.dtype)[: self.size].copy() if self.data is not None
                  else np.zeros(0, self.dtype))
        mask = None
        if self.mask is not None:
            mask = self.mask.cpu().numpy().view(np.uint32)[: (self.size + 31) // 32].copy()
        return HostFixedColumn(values, mask, self.size, self.null_count)


_DTYPES = {_capi.TYPE_INT32: np.dtype(np.int32), _capi.TYPE_UINT32: np.dtype(np.uint32),
           _capi.TYPE_UINT64: np.dtype(np.uint64)}


def _wrap(out: _capi.ListColumn) -> DeviceListColumn:
    mr = _mr()
    return DeviceListColumn(mr.take(out.offsets), mr.take(out.child), mr.take(out.null_mask),
                            int(out.size), int(out.null_count), _DTYPES[int(out.child_type)], int(out.child_size))


def _param_tensor(x, np_dtype):
    """a/b parameters: a device tensor (raw bits of uint32/uint64) or anything numpy can read."""
    torch = _torch()
    if isinstance(x, torch.Tensor):
        want = 4 if np_dtype == np.uint32 else 8
        if x.element_size() != want:
            raise TypeError(f"parameter tensor must have {want}-byte elements")
        return x.contiguous()
    arr = np.ascontiguousarray(x)
    if arr.dtype != np_dtype:
        raise TypeError(f"parameters must be {np.dtype(np_dtype).name}")
    signed = np.int32 if np_dtype == np.uint32 else np.int64
    return torch.from_numpy(arr.view(signed)).to("cuda")


def minhash(input: DeviceStringsColumn, seed: int, a, b, width: int) -> DeviceListColumn:
    """nvtext::minhash (cpp/include/nvtext/minhash.hpp:62-69); pylibcudf minhash.pyx:33-84."""
    L = _capi.load()
    if not (0 <= int(seed) < 2**32):
        raise ValueError("seed must fit uint32")
    ta, tb = _param_tensor(a, np.uint32), _param_tensor(b, np.uint32)
    out = _capi.ListColumn()
    col = input._c()
    st = L.nvtext_amd_minhash(C.byref(col), int(seed), ta.data_ptr() if ta.numel() else None,
                              tb.data_ptr() if tb.numel() else None, ta.numel(), tb.numel(), int(width),
                              _stream_handle(), C.byref(_mr().struct), C.byref(out))
    if st != _capi.SUCCESS:
        _raise(st)
    return _wrap(out)


MINHASH_PREALLOCATED_MAX_ROWS = 1048576  # NVTEXT_AMD_MINHASH_PREALLOCATED_MAX_ROWS


def minhash_preallocated(input: DeviceStringsColumn, seed: int, a, b, width: int, out_offsets, out_child, out_null_mask=None) -> None:
    """nvtext_amd_minhash_preallocated: minhash into buffers of the caller (int32 tensors of size + 1 and of at least
    (size - null_count) * len(a) values, and (size + 31) // 32 mask words when the input has a mask).  The call
    allocates nothing on the device; the parameters must already be device tensors."""
    L = _capi.load()
    if not (0 <= int(seed) < 2**32):
        raise ValueError("seed must fit uint32")
    col = input._c()
    st = L.nvtext_amd_minhash_preallocated(C.byref(col), int(seed), a.data_ptr() if a.numel() else None,
                                           b.data_ptr() if b.numel() else None, a.numel(), b.numel(), int(width), _stream_handle(),
                                           out_offsets.data_ptr(), out_child.data_ptr() if out_child.numel() else None,
                                           out_child.numel(), out_null_mask.data_ptr() if out_null_mask is not None else None)
    if st != _capi.SUCCESS:
        _raise(st)


def minhash64(input: DeviceStringsColumn, seed: int, a, b, width: int) -> DeviceListColumn:
    """nvtext::minhash64 (cpp/include/nvtext/minhash.hpp:109-116); pylibcudf minhash.pyx:88-141."""
    L = _capi.load()
    if not (0 <= int(seed) < 2**64):
        raise ValueError("seed must fit uint64")
    ta, tb = _param_tensor(a, np.uint64), _param_tensor(b, np.uint64)
    out = _capi.ListColumn()
    col = input._c()
    st = L.nvtext_amd_minhash64(C.byref(col), int(seed), ta.data_ptr() if ta.numel() else None,
                                tb.data_ptr() if tb.numel() else None, ta.numel(), tb.numel(), int(width),
                                _stream_handle(), C.byref(_mr().struct), C.byref(out))
    if st != _capi.SUCCESS:
        _raise(st)
    return _wrap(out)


def minhash_ngrams(input: DeviceListStringsColumn, ngrams: int, seed: int, a, b) -> DeviceListColumn:
    """nvtext::minhash_ngrams (cpp/include/nvtext/minhash.hpp:156-163); pylibcudf minhash.pyx minhash_ngrams."""
    L = _capi.load()
    if not (0 <= int(seed) < 2**32):
        raise ValueError("seed must fit uint32")
    ta, tb = _param_tensor(a, np.uint32), _param_tensor(b, np.uint32)
    out = _capi.ListColumn()
    col = input._c()
    st = L.nvtext_amd_minhash_ngrams(C.byref(col), int(ngrams), int(seed), ta.data_ptr() if ta.numel() else None,
                                     tb.data_ptr() if tb.numel() else None, ta.numel(), tb.numel(),
                                     _stream_handle(), C.byref(_mr().struct), C.byref(out))
    if st != _capi.SUCCESS:
        _raise(st)
    return _wrap(out)


def minhash64_ngrams(input: DeviceListStringsColumn, ngrams: int, seed: int, a, b) -> DeviceListColumn:
    """nvtext::minhash64_ngrams (cpp/include/nvtext/minhash.hpp:203-210); pylibcudf minhash.pyx minhash64_ngrams."""
    L = _capi.load()
    if not (0 <= int(seed) < 2**64):
        raise ValueError("seed must fit uint64")
    ta, tb = _param_tensor(a, np.uint64), _param_tensor(b, np.uint64)
    out = _capi.ListColumn()
    col = input._c()
    st = L.nvtext_amd_minhash64_ngrams(C.byref(col), int(ngrams), int(seed), ta.data_ptr() if ta.numel() else None,
                                       tb.data_ptr() if tb.numel() else None, ta.numel(), tb.numel(),
                                       _stream_handle(), C.byref(_mr().struct), C.byref(out))
    if st != _capi.SUCCESS:
        _raise(st)
    return _wrap(out)


def jaccard_index(input1: DeviceStringsColumn, input2: DeviceStringsColumn, width: int) -> DeviceFixedColumn:
    """nvtext::jaccard_index (cpp/include/nvtext/jaccard.hpp:66-71); pylibcudf jaccard.pyx jaccard_index."""
    L = _capi.load()
    out = _capi.FixedColumn()
    c1, c2 = input1._c(), input2._c()
    st = L.nvtext_amd_jaccard_index(C.byref(c1), C.byref(c2), int(width), _stream_handle(), C.byref(_mr().struct), C.byref(out))
    if st != _capi.SUCCESS:
        _raise(st)
    mr = _mr()
    return DeviceFixedColumn(mr.take(out.data), mr.take(out.null_mask), int(out.size), int(out.null_count), np.dtype(np.float32))


class CharacterNormalizer:
    """nvtext::character_normalizer (cpp/include/nvtext/normalize.hpp:81-124); pylibcudf normalize.pyx CharacterNormalizer."""

    def __init__(self, do_lower_case: bool, special_tokens: Optional[DeviceStringsColumn] = None):
        L = _capi.load()
        h = C.c_void_p()
        col = special_tokens._c() if special_tokens is not None else None
        st = L.nvtext_amd_character_normalizer_create(int(bool(do_lower_case)), C.byref(col) if col is not None else None,
                                                      _stream_handle(), C.byref(_mr().struct), C.byref(h))
        if st != _capi.SUCCESS:
            _raise(st)
        self._h = h
        self.do_lower_case = bool(do_lower_case)

    def __del__(self, _finalizing=sys.is_finalizing):
        # the tables go back through the allocator's callback into Python: not while the interpreter is shutting down
        # (when this module's globals may be gone already, hence the default argument)
        h, self._h = getattr(self, "_h", None), None
        if h and not _finalizing():
            try:
                _capi.load().nvtext_amd_character_normalizer_destroy(h)
            except Exception:
                pass


def normalize_characters(input: DeviceStringsColumn, normalizer: CharacterNormalizer) -> DeviceStringsColumn:
    """nvtext::normalize_characters (cpp/include/nvtext/normalize.hpp:126-160); pylibcudf normalize.pyx normalize_characters."""
    L = _capi.load()
    out = _capi.StringsResult()
    col = input._c()
    st = L.nvtext_amd_normalize_characters(C.byref(col), normalizer._h, _stream_handle(), C.byref(_mr().struct), C.byref(out))
    if st != _capi.SUCCESS:
        _raise(st)
    mr = _mr()
    torch = _torch()
    chars = mr.take(out.chars)
    offsets = mr.take(out.offsets)
    mask = mr.take(out.null_mask)
    if chars is None:
        chars = torch.empty(0, dtype=torch.uint8, device="cuda")
    else:
        chars = chars[: int(out.chars_size)]
    if offsets is not None:
        offsets = offsets.view(torch.int64 if out.offsets_is_int64 else torch.int32)[: int(out.offsets_size)]
    if mask is not None:
        mask = mask[: (int(out.size) + 31) // 32 * 4].view(torch.int32)
    return DeviceStringsColumn(chars, offsets, mask, int(out.size), 0, int(out.null_count))


class WordPieceVocabulary:
    """nvtext::wordpiece_vocabulary (cpp/include/nvtext/wordpiece_tokenize.hpp:26-66);
    pylibcudf wordpiece_tokenize.pyx:22-47."""

    def __init__(self, vocab: DeviceStringsColumn):
        L = _capi.load()
        h = C.c_void_p()
        col = vocab._c()
        st = L.nvtext_amd_wordpiece_vocabulary_create(C.byref(col), _stream_handle(), C.byref(_mr().struct), C.byref(h))
        if st != _capi.SUCCESS:
            _raise(st)
        self._h = h
        self.unk_id = int(L.nvtext_amd_wordpiece_vocabulary_unk_id(h))

    def __del__(self, _finalizing=sys.is_finalizing):
        # the tables go back through the allocator's callback into Python: not while the interpreter is shutting down
        # (when this module's globals may be gone already, hence the default argument)
        h, self._h = getattr(self, "_h", None), None
        if h and not _finalizing():
            try:
                _capi.load().nvtext_amd_wordpiece_vocabulary_destroy(h)
            except Exception:
                pass


def wordpiece_tokenize(input: DeviceStringsColumn, vocabulary: WordPieceVocabulary, max_words_per_row: int = 0) -> DeviceListColumn:
    """nvtext::wordpiece_tokenize (cpp/include/nvtext/wordpiece_tokenize.hpp:68-111);
    pylibcudf wordpiece_tokenize.pyx:51-97."""
    L = _capi.load()
    out = _capi.ListColumn()
    col = input._c()
    st = L.nvtext_amd_wordpiece_tokenize(C.byref(col), vocabulary._h, int(max_words_per_row), _stream_handle(),
                                         C.byref(_mr().struct), C.byref(out))
    if st != _capi.SUCCESS:
        _raise(st)
    return _wrap(out)
