"""Host-side Arrow-layout strings / list columns (numpy buffers).

Layout follows libcudf's strings column
(cpp/include/cudf/strings/strings_column_view.hpp:27-114): a chars buffer, an
offsets child (int32 or int64) and an optional validity bitmask of uint32 words
with bit ``i`` (LSB first) describing row ``i`` (cpp/include/cudf/utilities/bit.hpp:101-105).
A sliced view keeps the parent's buffers and carries ``offset``/``size``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, List, Optional, Sequence, Union

import numpy as np

Text = Union[str, bytes, None]


def mask_words(nbits: int) -> int:
    return (nbits + 31) // 32


def pack_validity(valid: Sequence[bool]) -> np.ndarray:
    """bool[rows] -> uint32 words, LSB-first."""
    valid = np.asarray(valid, dtype=bool)
    n = valid.size
    padded = np.zeros(mask_words(n) * 32, dtype=np.uint8)
    padded[:n] = valid
    return np.packbits(padded, bitorder="little").view(np.uint32).copy()


def unpack_validity(mask: np.ndarray, size: int, offset: int = 0) -> np.ndarray:
    bits = np.unpackbits(np.ascontiguousarray(mask).view(np.uint8), bitorder="little")
    return bits[offset:offset + size].astype(bool)


@dataclass
class HostStringsColumn:
    chars: np.ndarray            # uint8
    offsets: np.ndarray          # int32 or int64, parent_size + 1 entries
    mask: Optional[np.ndarray]   # uint32 words or None
    size: int
    offset: int = 0
    null_count: int = 0

    @staticmethod
    def from_pylist(rows: Iterable[Text], offsets_dtype=np.int32, force_mask: bool = False) -> "HostStringsColumn":
        """Null rows become zero-length, as cudf::test::strings_column_wrapper does
        (cpp/include/cudf_test/column_wrapper.hpp:325-339)."""
        enc: List[bytes] = []
        valid: List[bool] = []
        for r in rows:
            if r is None:
                enc.append(b"")
                valid.append(False)
            else:
                enc.append(r.encode("utf-8") if isinstance(r, str) else bytes(r))
                valid.append(True)
        n = len(enc)
        offsets = np.zeros(n + 1, dtype=np.int64)
        if n:
            np.cumsum([len(e) for e in enc], out=offsets[1:])
        chars = np.frombuffer(b"".join(enc), dtype=np.uint8).copy() if n else np.zeros(0, np.uint8)
        nulls = n - int(sum(valid))
        mask = pack_validity(valid) if (nulls or force_mask) and n else None
        return HostStringsColumn(chars, offsets.astype(offsets_dtype), mask, n, 0, nulls)

    def slice(self, lo: int, hi: int) -> "HostStringsColumn":
        """cudf::slice semantics: same buffers, new offset/size, null count recomputed."""
        assert 0 <= lo <= hi <= self.size
        nulls = 0
        if self.mask is not None:
            nulls = int((~unpack_validity(self.mask, hi - lo, self.offset + lo)).sum())
        return HostStringsColumn(self.chars, self.offsets, self.mask, hi - lo, self.offset + lo, nulls)

    def validity(self) -> np.ndarray:
        if self.mask is None:
            return np.ones(self.size, dtype=bool)
        return unpack_validity(self.mask, self.size, self.offset)

    def to_pylist(self) -> List[Optional[bytes]]:
        v = self.validity()
        out: List[Optional[bytes]] = []
        for i in range(self.size):
            if not v[i]:
                out.append(None)
                continue
            b, e = int(self.offsets[self.offset + i]), int(self.offsets[self.offset + i + 1])
            out.append(self.chars[b:e].tobytes())
        return out

    @property
    def chars_bytes(self) -> int:
        if self.size == 0 or self.offsets.size == 0:
            return 0
        return int(self.offsets[self.offset + self.size]) - int(self.offsets[self.offset])


@dataclass
class HostListStringsColumn:
    """LIST<STRING> column (cpp/include/cudf/lists/lists_column_view.hpp): int32 list offsets
    (parent_size + 1 entries, element indices into the child), an optional row validity mask, and a
    strings child.  A sliced view keeps the buffers and carries ``offset``/``size``."""
    offsets: np.ndarray          # int32
    child: HostStringsColumn
    mask: Optional[np.ndarray]
    size: int
    offset: int = 0
    null_count: int = 0

    @staticmethod
    def from_pylist(rows, child_offsets_dtype=np.int32) -> "HostListStringsColumn":
        """rows: list of (list of str/bytes/None) or None.  Null rows are empty lists, as
        cudf::test::lists_column_wrapper builds them."""
        flat: List[Text] = []
        offs = [0]
        valid = []
        for r in rows:
            if r is None:
                valid.append(False)
            else:
                valid.append(True)
                flat.extend(r)
            offs.append(len(flat))
        n = len(valid)
        nulls = n - int(sum(valid))
        child = HostStringsColumn.from_pylist(flat, child_offsets_dtype)
        mask = pack_validity(valid) if nulls and n else None
        return HostListStringsColumn(np.asarray(offs, dtype=np.int32), child, mask, n, 0, nulls)

    def slice(self, lo: int, hi: int) -> "HostListStringsColumn":
        assert 0 <= lo <= hi <= self.size
        nulls = 0
        if self.mask is not None:
            nulls = int((~unpack_validity(self.mask, hi - lo, self.offset + lo)).sum())
        return HostListStringsColumn(self.offsets, self.child, self.mask, hi - lo, self.offset + lo, nulls)

    def validity(self) -> np.ndarray:
        if self.mask is None:
            return np.ones(self.size, dtype=bool)
        return unpack_validity(self.mask, self.size, self.offset)


@dataclass
class HostFixedColumn:
    """Fixed-width column (here FLOAT32 results): values, optional validity mask."""
    values: np.ndarray
    mask: Optional[np.ndarray]
    size: int
    null_count: int = 0

    def validity(self) -> np.ndarray:
        if self.mask is None:
            return np.ones(self.size, dtype=bool)
        return unpack_validity(self.mask, self.size, 0)

    def to_pylist(self):
        v = self.validity()
        return [self.values[i].item() if v[i] else None for i in range(self.size)]

    def equals(self, other: "HostFixedColumn") -> bool:
        """Size, null count, validity and the bits of every valid value."""
        if self.size != other.size or self.null_count != other.null_count or self.values.dtype != other.values.dtype:
            return False
        v = self.validity()
        if not np.array_equal(v, other.validity()):
            return False
        a = np.ascontiguousarray(self.values[: self.size]).view(np.uint32)
        b = np.ascontiguousarray(other.values[: other.size]).view(np.uint32)
        return bool(np.array_equal(a[v], b[v]))


@dataclass
class HostListColumn:
    """LIST<INT32|UINT32|UINT64> result (cpp/src/lists/lists_column_factories.cu:106-129):
    int32 offsets (size+1 entries, or 0 entries for the canonical empty list column),
    a non-nullable child and an optional validity mask."""
    offsets: np.ndarray
    child: np.ndarray
    mask: Optional[np.ndarray]
    size: int
    null_count: int = 0

    def validity(self) -> np.ndarray:
        if self.mask is None:
            return np.ones(self.size, dtype=bool)
        return unpack_validity(self.mask, self.size, 0)

    def to_pylist(self) -> List[Optional[List[int]]]:
        v = self.validity()
        out: List[Optional[List[int]]] = []
        for i in range(self.size):
            if not v[i]:
                out.append(None)
            else:
                out.append(self.child[int(self.offsets[i]):int(self.offsets[i + 1])].tolist())
        return out

    def equals(self, other: "HostListColumn") -> bool:
        """Exact comparison in the spirit of CUDF_TEST_EXPECT_COLUMNS_EQUAL
        (cpp/include/cudf_test/column_utilities.hpp:288-292): size, null count,
        validity bits, offsets and child values."""
        if self.size != other.size or self.null_count != other.null_count:
            return False
        if self.child.dtype != other.child.dtype:
            return False
        if not np.array_equal(self.validity(), other.validity()):
            return False
        if self.offsets.size != other.offsets.size:
            return False
        return bool(np.array_equal(self.offsets, other.offsets) and np.array_equal(self.child, other.child))
