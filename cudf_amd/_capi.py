"""ctypes declarations for the C ABI in include/nvtext_amd.h (libnvtext_amd.so)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# NVTEXT_AMD_LIB names another build of the library (experiments; the default is the in-tree build)
LIB_PATH = os.environ.get("NVTEXT_AMD_LIB") or os.path.join(_HERE, "libnvtext_amd.so")

SUCCESS, INVALID_ARGUMENT, OVERFLOW, LOGIC_ERROR, DEVICE_ERROR, ALLOC_FAILED = range(6)
TYPE_INT32, TYPE_UINT32, TYPE_UINT64, TYPE_FLOAT32 = 3, 7, 8, 9

EXPORTS = [
    "nvtext_amd_version",
    "nvtext_amd_last_error",
    "nvtext_amd_minhash",
    "nvtext_amd_minhash64",
    "nvtext_amd_minhash_preallocated",
    "nvtext_amd_minhash_ngrams",
    "nvtext_amd_minhash64_ngrams",
    "nvtext_amd_jaccard_index",
    "nvtext_amd_fixed_column_free",
    "nvtext_amd_strings_from_arrow_device",
    "nvtext_amd_list_strings_from_arrow_device",
    "nvtext_amd_list_to_arrow_device",
    "nvtext_amd_fixed_to_arrow_device",
    "nvtext_amd_strings_to_arrow_device",
    "nvtext_amd_character_normalizer_create",
    "nvtext_amd_character_normalizer_destroy",
    "nvtext_amd_normalize_characters",
    "nvtext_amd_strings_result_free",
    "nvtext_amd_wordpiece_vocabulary_create",
    "nvtext_amd_wordpiece_vocabulary_destroy",
    "nvtext_amd_wordpiece_vocabulary_unk_id",
    "nvtext_amd_wordpiece_tokenize",
    "nvtext_amd_list_column_free",
    "nvtext_amd_profile_enable",
    "nvtext_amd_profile_read",
    "nvtext_amd_profile_set_range_tiles",
    "nvtext_amd_profile_set_sizing_sample",
]


class StringsColumn(C.Structure):
    _fields_ = [
        ("chars", C.c_void_p),
        ("offsets", C.c_void_p),
        ("offsets_is_int64", C.c_int32),
        ("null_mask", C.c_void_p),
        ("size", C.c_int32),
        ("offset", C.c_int32),
        ("null_count", C.c_int32),
    ]


class ListStringsColumn(C.Structure):
    _fields_ = [
        ("offsets", C.c_void_p),
        ("null_mask", C.c_void_p),
        ("size", C.c_int32),
        ("offset", C.c_int32),
        ("null_count", C.c_int32),
        ("child", StringsColumn),
    ]


ALLOC_FN = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p)
DEALLOC_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p)


class Allocator(C.Structure):
    _fields_ = [("ctx", C.c_void_p), ("allocate", ALLOC_FN), ("deallocate", DEALLOC_FN)]


class ListColumn(C.Structure):
    _fields_ = [
        ("size", C.c_int32),
        ("null_count", C.c_int32),
        ("child_type", C.c_int32),
        ("offsets_size", C.c_int32),
        ("offsets", C.c_void_p),
        ("child", C.c_void_p),
        ("child_size", C.c_int64),
        ("null_mask", C.c_void_p),
        ("offsets_bytes", C.c_size_t),
        ("child_bytes", C.c_size_t),
        ("null_mask_bytes", C.c_size_t),
    ]


class FixedColumn(C.Structure):
    _fields_ = [
        ("type", C.c_int32),
        ("size", C.c_int32),
        ("null_count", C.c_int32),
        ("data", C.c_void_p),
        ("null_mask", C.c_void_p),
        ("data_bytes", C.c_size_t),
        ("null_mask_bytes", C.c_size_t),
    ]


class StringsResult(C.Structure):
    _fields_ = [
        ("size", C.c_int32),
        ("null_count", C.c_int32),
        ("offsets_size", C.c_int32),
        ("offsets_is_int64", C.c_int32),
        ("offsets", C.c_void_p),
        ("chars", C.c_void_p),
        ("chars_size", C.c_int64),
        ("null_mask", C.c_void_p),
        ("offsets_bytes", C.c_size_t),
        ("chars_bytes", C.c_size_t),
        ("null_mask_bytes", C.c_size_t),
    ]


# ---- Arrow C data / device interface (arrow/c/abi.h)
class ArrowSchema(C.Structure):
    pass


ArrowSchema._fields_ = [
    ("format", C.c_char_p), ("name", C.c_char_p), ("metadata", C.c_char_p), ("flags", C.c_int64), ("n_children", C.c_int64),
    ("children", C.POINTER(C.POINTER(ArrowSchema))), ("dictionary", C.POINTER(ArrowSchema)),
    ("release", C.CFUNCTYPE(None, C.POINTER(ArrowSchema))), ("private_data", C.c_void_p)]


class ArrowArray(C.Structure):
    pass


ArrowArray._fields_ = [
    ("length", C.c_int64), ("null_count", C.c_int64), ("offset", C.c_int64), ("n_buffers", C.c_int64), ("n_children", C.c_int64),
    ("buffers", C.POINTER(C.c_void_p)), ("children", C.POINTER(C.POINTER(ArrowArray))), ("dictionary", C.POINTER(ArrowArray)),
    ("release", C.CFUNCTYPE(None, C.POINTER(ArrowArray))), ("private_data", C.c_void_p)]


class ArrowDeviceArray(C.Structure):
    _fields_ = [("array", ArrowArray), ("device_id", C.c_int64), ("device_type", C.c_int32), ("sync_event", C.c_void_p),
                ("reserved", C.c_int64 * 3)]


ARROW_DEVICE_CPU, ARROW_DEVICE_ROCM, ARROW_DEVICE_ROCM_HOST = 1, 10, 11
ARROW_FLAG_NULLABLE = 2

_lib = None


class ExtensionMissing(RuntimeError):
    pass


def _share_the_hip_runtime_of_torch():
    """A process must hold ONE HIP runtime: of two, the one that initialises second finds no device.  torch's wheels
    bring their own libamdhip64 and load it when torch first touches the GPU; the library names its runtime by soname
    (libamdhip64.so.7) and would take the system's if none is loaded yet.  The device buffers of this host side are
    torch's, so torch's runtime is loaded first, and the library's dependency then resolves to it.  (A caller without
    torch, like tests/cpp/nvtext_api_test.cpp, has the system's runtime alone.)"""
    try:
        import torch
    except ImportError:
        return
    bundled = os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so")
    if os.path.exists(bundled):
        C.CDLL(bundled, mode=C.RTLD_GLOBAL)


def load():
    """Loads the HIP library.  There is no fallback: without it the package cannot compute."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ExtensionMissing(
            f"{LIB_PATH} is missing: build it with `make -C cudf_amd/csrc` (or __graft_entry__.build())")
    _share_the_hip_runtime_of_torch()
    L = C.CDLL(LIB_PATH)
    L.nvtext_amd_version.restype = C.c_int32
    L.nvtext_amd_version.argtypes = []
    L.nvtext_amd_last_error.restype = C.c_char_p
    L.nvtext_amd_last_error.argtypes = []
    common_tail = [C.c_int32, C.c_void_p, C.POINTER(Allocator), C.POINTER(ListColumn)]
    L.nvtext_amd_minhash.restype = C.c_int
    L.nvtext_amd_minhash.argtypes = [C.POINTER(StringsColumn), C.c_uint32, C.c_void_p, C.c_void_p,
                                     C.c_int64, C.c_int64] + common_tail
    L.nvtext_amd_minhash_preallocated.restype = C.c_int
    L.nvtext_amd_minhash_preallocated.argtypes = [C.POINTER(StringsColumn), C.c_uint32, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                                  C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
    L.nvtext_amd_minhash64.restype = C.c_int
    L.nvtext_amd_minhash64.argtypes = [C.POINTER(StringsColumn), C.c_uint64, C.c_void_p, C.c_void_p,
                                       C.c_int64, C.c_int64] + common_tail
    L.nvtext_amd_minhash_ngrams.restype = C.c_int
    L.nvtext_amd_minhash_ngrams.argtypes = [C.POINTER(ListStringsColumn), C.c_int32, C.c_uint32, C.c_void_p, C.c_void_p,
                                            C.c_int64, C.c_int64] + common_tail[1:]
    L.nvtext_amd_minhash64_ngrams.restype = C.c_int
    L.nvtext_amd_minhash64_ngrams.argtypes = [C.POINTER(ListStringsColumn), C.c_int32, C.c_uint64, C.c_void_p, C.c_void_p,
                                              C.c_int64, C.c_int64] + common_tail[1:]
    L.nvtext_amd_jaccard_index.restype = C.c_int
    L.nvtext_amd_jaccard_index.argtypes = [C.POINTER(StringsColumn), C.POINTER(StringsColumn), C.c_int32, C.c_void_p,
                                           C.POINTER(Allocator), C.POINTER(FixedColumn)]
    L.nvtext_amd_fixed_column_free.restype = None
    L.nvtext_amd_fixed_column_free.argtypes = [C.POINTER(FixedColumn), C.c_void_p, C.POINTER(Allocator)]
    L.nvtext_amd_strings_from_arrow_device.restype = C.c_int
    L.nvtext_amd_strings_from_arrow_device.argtypes = [C.POINTER(ArrowSchema), C.POINTER(ArrowDeviceArray), C.c_void_p, C.POINTER(StringsColumn)]
    L.nvtext_amd_list_strings_from_arrow_device.restype = C.c_int
    L.nvtext_amd_list_strings_from_arrow_device.argtypes = [C.POINTER(ArrowSchema), C.POINTER(ArrowDeviceArray), C.c_void_p,
                                                            C.POINTER(ListStringsColumn)]
    L.nvtext_amd_list_to_arrow_device.restype = C.c_int
    L.nvtext_amd_list_to_arrow_device.argtypes = [C.POINTER(ListColumn), C.c_void_p, C.POINTER(Allocator), C.POINTER(ArrowSchema),
                                                  C.POINTER(ArrowDeviceArray)]
    L.nvtext_amd_fixed_to_arrow_device.restype = C.c_int
    L.nvtext_amd_fixed_to_arrow_device.argtypes = [C.POINTER(FixedColumn), C.c_void_p, C.POINTER(Allocator), C.POINTER(ArrowSchema),
                                                   C.POINTER(ArrowDeviceArray)]
    L.nvtext_amd_strings_to_arrow_device.restype = C.c_int
    L.nvtext_amd_strings_to_arrow_device.argtypes = [C.POINTER(StringsResult), C.c_void_p, C.POINTER(Allocator), C.POINTER(ArrowSchema),
                                                     C.POINTER(ArrowDeviceArray)]
    L.nvtext_amd_character_normalizer_create.restype = C.c_int
    L.nvtext_amd_character_normalizer_create.argtypes = [C.c_int32, C.POINTER(StringsColumn), C.c_void_p, C.POINTER(Allocator),
                                                         C.POINTER(C.c_void_p)]
    L.nvtext_amd_character_normalizer_destroy.restype = None
    L.nvtext_amd_character_normalizer_destroy.argtypes = [C.c_void_p]
    L.nvtext_amd_normalize_characters.restype = C.c_int
    L.nvtext_amd_normalize_characters.argtypes = [C.POINTER(StringsColumn), C.c_void_p, C.c_void_p, C.POINTER(Allocator),
                                                  C.POINTER(StringsResult)]
    L.nvtext_amd_strings_result_free.restype = None
    L.nvtext_amd_strings_result_free.argtypes = [C.POINTER(StringsResult), C.c_void_p, C.POINTER(Allocator)]
    L.nvtext_amd_wordpiece_vocabulary_create.restype = C.c_int
    L.nvtext_amd_wordpiece_vocabulary_create.argtypes = [C.POINTER(StringsColumn), C.c_void_p,
                                                         C.POINTER(Allocator), C.POINTER(C.c_void_p)]
    L.nvtext_amd_wordpiece_vocabulary_destroy.restype = None
    L.nvtext_amd_wordpiece_vocabulary_destroy.argtypes = [C.c_void_p]
    L.nvtext_amd_wordpiece_vocabulary_unk_id.restype = C.c_int32
    L.nvtext_amd_wordpiece_vocabulary_unk_id.argtypes = [C.c_void_p]
    L.nvtext_amd_wordpiece_tokenize.restype = C.c_int
    L.nvtext_amd_wordpiece_tokenize.argtypes = [C.POINTER(StringsColumn), C.c_void_p] + common_tail
    L.nvtext_amd_list_column_free.restype = None
    L.nvtext_amd_list_column_free.argtypes = [C.POINTER(ListColumn), C.c_void_p, C.POINTER(Allocator)]
    L.nvtext_amd_profile_enable.restype = None
    L.nvtext_amd_profile_enable.argtypes = [C.c_int32]
    L.nvtext_amd_profile_read.restype = C.c_int32
    L.nvtext_amd_profile_read.argtypes = [C.POINTER(C.c_char_p), C.POINTER(C.c_float), C.c_int32]
    L.nvtext_amd_profile_set_range_tiles.restype = None
    L.nvtext_amd_profile_set_range_tiles.argtypes = [C.c_int32]
    L.nvtext_amd_profile_set_sizing_sample.restype = None
    L.nvtext_amd_profile_set_sizing_sample.argtypes = [C.c_int32]
    _lib = L
    return L


def profile_enable(on: bool) -> None:
    load().nvtext_amd_profile_enable(1 if on else 0)


def set_range_tiles(tiles: int) -> None:
    """Test knob: ranges of `tiles` (1, 2, 4, 8) tiles in every later wordpiece_tokenize call; 0 = sized by the column."""
    load().nvtext_amd_profile_set_range_tiles(int(tiles))


def set_sizing_sample(on: bool) -> None:
    """Test knob: whether wordpiece_tokenize sizes its first attempt from a sample of the column (the default)."""
    load().nvtext_amd_profile_set_sizing_sample(1 if on else 0)


def profile_read(capacity: int = 4096):
    """[(kernel name, milliseconds)] in launch order since the last read."""
    names = (C.c_char_p * capacity)()
    ms = (C.c_float * capacity)()
    n = load().nvtext_amd_profile_read(names, ms, capacity)
    return [(names[i].decode(), float(ms[i])) for i in range(n)]
