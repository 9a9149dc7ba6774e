"""Arrow C Device Data Interface adaptors (include/nvtext_amd_arrow.h), driven through the C ABI.

Inputs are built with pyarrow on the host, their buffers copied to the GPU and described by a hand-made
ArrowDeviceArray (pyarrow here cannot allocate ROCm memory).  Results come back as ArrowDeviceArrays; their
buffers are copied to the host and handed, with the schema the library exported, to pyarrow's own importer,
which therefore checks formats, children, flags and buffer layout; values are compared with the oracle.
"""
import ctypes as C

import numpy as np
import pytest

pa = pytest.importorskip("pyarrow")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cudf_amd import _capi, nvtext
    from oracle import pyoracle
    return dict(torch=torch, capi=_capi, lib=_capi.load(), nv=nvtext, orc=pyoracle, mr=nvtext._mr(), keep=[])


def stream_of(env):
    return int(env["torch"].cuda.current_stream().cuda_stream)


def device_copy(env, buf):
    """pyarrow buffer -> device tensor (kept alive by the caller); None stays None."""
    if buf is None:
        return None
    host = np.frombuffer(buf, dtype=np.uint8)
    padded = np.zeros((host.size + 15) // 16 * 16 + 16, np.uint8)
    padded[: host.size] = host
    t = env["torch"].from_numpy(padded).cuda()
    env["keep"].append(t)
    return t


def export_schema(env, typ):
    s = env["capi"].ArrowSchema()
    typ._export_to_c(C.addressof(s))
    return s


def device_array_of(env, arr, device_type=None, null_count=None):
    """An ArrowDeviceArray over device copies of the buffers of the pyarrow array (children too)."""
    capi = env["capi"]

    def fill(a, target):
        bufs = [device_copy(env, b) for b in a.buffers()[: {True: 2, False: 3}[pa.types.is_list(a.type)]]]
        ptrs = (C.c_void_p * len(bufs))(*[t.data_ptr() if t is not None else None for t in bufs])
        env["keep"].append(ptrs)
        target.length, target.offset = len(a), a.offset
        target.null_count = a.null_count if null_count is None else null_count
        target.n_buffers, target.buffers = len(bufs), ptrs
        target.n_children = 0
        if pa.types.is_list(a.type):
            child = capi.ArrowArray()
            fill(a.values, child)  # the whole child array, as the C data interface exports it
            kids = (C.POINTER(capi.ArrowArray) * 1)(C.pointer(child))
            env["keep"] += [child, kids]
            target.n_children, target.children = 1, kids

    d = capi.ArrowDeviceArray()
    fill(arr, d.array)
    d.device_id = 0
    d.device_type = capi.ARROW_DEVICE_ROCM if device_type is None else device_type
    d.sync_event = None
    return d


def host_strings(arr):
    """The same column for the oracle (cudf_amd.arrow_host.HostStringsColumn over the array's own buffers)."""
    from cudf_amd.arrow_host import HostStringsColumn
    validity, offsets, data = arr.buffers()
    odt = np.int64 if pa.types.is_large_string(arr.type) else np.int32
    off = np.frombuffer(offsets, dtype=odt)
    chars = np.frombuffer(data, dtype=np.uint8) if data is not None else np.zeros(0, np.uint8)
    mask = None
    if validity is not None:
        raw = np.frombuffer(validity, dtype=np.uint8)
        padded = np.zeros((raw.size + 3) // 4 * 4, np.uint8)
        padded[: raw.size] = raw
        mask = padded.view(np.uint32)
    return HostStringsColumn(chars, off, mask, len(arr), arr.offset, arr.null_count)


def import_result(env, schema, darr):
    """Copies the buffers of a result ArrowDeviceArray to the host and lets pyarrow import the host mirror together with
    the schema the library exported.  Returns the pyarrow array."""
    capi = env["capi"]
    assert darr.device_type == capi.ARROW_DEVICE_ROCM and darr.sync_event
    env["torch"].cuda.synchronize()
    live = env["mr"].live
    keep = []

    release_type = C.CFUNCTYPE(None, C.POINTER(capi.ArrowArray))

    @release_type
    def release_mirror(p):
        p.contents.release = release_type()

    keep.append(release_mirror)

    def mirror(src):
        dst = capi.ArrowArray()
        dst.length, dst.null_count, dst.offset = src.length, src.null_count, src.offset
        dst.n_buffers, dst.n_children = src.n_buffers, src.n_children
        ptrs = (C.c_void_p * src.n_buffers)()
        for i in range(src.n_buffers):
            p = src.buffers[i]
            if p:
                host = live[p].cpu().numpy().copy()  # the allocator still owns the buffer until release
                keep.append(host)
                ptrs[i] = host.ctypes.data
        dst.buffers = ptrs
        keep.append(ptrs)
        if src.n_children:
            kid = mirror(src.children[0].contents)
            kids = (C.POINTER(capi.ArrowArray) * 1)(C.pointer(kid))
            keep.extend([kid, kids])
            dst.children = kids
        dst.release = release_mirror
        return dst

    m = mirror(darr.array)
    out = pa.Array._import_from_c(C.addressof(m), C.addressof(schema))
    assert not schema.release  # pyarrow moved the schema out: the library's release callback is pyarrow's business now
    copy = pa.array(out.to_pylist(), type=out.type)  # detach from the mirrors before they go out of scope
    del out
    return copy, keep


@pytest.mark.parametrize("typ", [pa.string(), pa.large_string()], ids=["utf8", "large_utf8"])
@pytest.mark.parametrize("unknown_nulls", [False, True])
def test_minhash_arrow_in_arrow_out(env, typ, unknown_nulls):
    capi, lib, orc = env["capi"], env["lib"], env["orc"]
    rng = np.random.default_rng(8)
    rows = [None if rng.random() < 0.1 else "".join(rng.choice(list("abcdé "), int(rng.integers(0, 60)))) for _ in range(500)]
    arr = pa.array(rows, type=typ).slice(7, 480)
    schema = export_schema(env, typ)
    darr = device_array_of(env, arr, null_count=-1 if unknown_nulls else None)
    col = capi.StringsColumn()
    assert lib.nvtext_amd_strings_from_arrow_device(C.byref(schema), C.byref(darr), stream_of(env), C.byref(col)) == capi.SUCCESS
    assert (col.size, col.offset, col.null_count) == (480, 7, arr.null_count)
    assert col.offsets_is_int64 == int(pa.types.is_large_string(typ))

    a = np.arange(3, 8, dtype=np.uint32)
    ta = env["torch"].from_numpy(a.view(np.int32)).cuda()
    out = capi.ListColumn()
    st = lib.nvtext_amd_minhash(C.byref(col), 11, ta.data_ptr(), ta.data_ptr(), 5, 5, 4, stream_of(env), C.byref(env["mr"].struct), C.byref(out))
    assert st == capi.SUCCESS
    offsets_ptr = out.offsets
    out_schema, out_arr = capi.ArrowSchema(), capi.ArrowDeviceArray()
    st = lib.nvtext_amd_list_to_arrow_device(C.byref(out), stream_of(env), C.byref(env["mr"].struct), C.byref(out_schema), C.byref(out_arr))
    assert st == capi.SUCCESS and not out.offsets and out.size == 0  # moved out
    got, keep = import_result(env, out_schema, out_arr)
    assert got.type == pa.list_(pa.field("element", pa.uint32(), nullable=False)) and got.null_count == arr.null_count
    exp = orc.minhash(host_strings(arr), 11, a, a, 4)
    assert got.to_pylist() == exp.to_pylist()
    # releasing the array hands the buffers back to the allocator they came from
    assert offsets_ptr in env["mr"].live
    out_arr.array.release(C.byref(out_arr.array))
    assert offsets_ptr not in env["mr"].live and not out_arr.array.release


def test_ngrams_and_jaccard_through_arrow(env):
    capi, lib, orc = env["capi"], env["lib"], env["orc"]
    from cudf_amd.arrow_host import HostListStringsColumn
    rng = np.random.default_rng(9)
    words = lambda n: ["".join(rng.choice(list("abc"), int(rng.integers(1, 6)))) for _ in range(n)]
    rows = [None if rng.random() < 0.1 else words(int(rng.integers(0, 30))) for _ in range(200)]
    typ = pa.list_(pa.string())
    arr = pa.array(rows, type=typ)
    schema = export_schema(env, typ)
    darr = device_array_of(env, arr)
    lcol = capi.ListStringsColumn()
    assert lib.nvtext_amd_list_strings_from_arrow_device(C.byref(schema), C.byref(darr), stream_of(env), C.byref(lcol)) == capi.SUCCESS
    a = np.arange(1, 4, dtype=np.uint64)
    ta = env["torch"].from_numpy(a.view(np.int64)).cuda()
    out = capi.ListColumn()
    st = lib.nvtext_amd_minhash64_ngrams(C.byref(lcol), 3, 5, ta.data_ptr(), ta.data_ptr(), 3, 3, stream_of(env), C.byref(env["mr"].struct), C.byref(out))
    assert st == capi.SUCCESS
    out_schema, out_arr = capi.ArrowSchema(), capi.ArrowDeviceArray()
    assert lib.nvtext_amd_list_to_arrow_device(C.byref(out), stream_of(env), C.byref(env["mr"].struct), C.byref(out_schema), C.byref(out_arr)) == capi.SUCCESS
    got, keep = import_result(env, out_schema, out_arr)
    exp = orc.minhash64_ngrams(HostListStringsColumn.from_pylist(rows), 3, 5, a, a)
    assert got.type == pa.list_(pa.field("element", pa.uint64(), nullable=False)) and got.to_pylist() == exp.to_pylist()
    out_arr.array.release(C.byref(out_arr.array))

    # jaccard_index: two utf8 arrays in, a float32 array out
    r1 = [None if rng.random() < 0.1 else " ".join(words(int(rng.integers(0, 20)))) for _ in range(300)]
    r2 = [None if rng.random() < 0.1 else " ".join(words(int(rng.integers(0, 20)))) for _ in range(300)]
    a1, a2 = pa.array(r1, type=pa.string()), pa.array(r2, type=pa.string())
    s = export_schema(env, pa.string())
    s2 = export_schema(env, pa.string())
    d1, d2 = device_array_of(env, a1), device_array_of(env, a2)
    c1, c2 = capi.StringsColumn(), capi.StringsColumn()
    assert lib.nvtext_amd_strings_from_arrow_device(C.byref(s), C.byref(d1), stream_of(env), C.byref(c1)) == capi.SUCCESS
    assert lib.nvtext_amd_strings_from_arrow_device(C.byref(s2), C.byref(d2), stream_of(env), C.byref(c2)) == capi.SUCCESS
    fixed = capi.FixedColumn()
    assert lib.nvtext_amd_jaccard_index(C.byref(c1), C.byref(c2), 3, stream_of(env), C.byref(env["mr"].struct), C.byref(fixed)) == capi.SUCCESS
    fs, fa = capi.ArrowSchema(), capi.ArrowDeviceArray()
    assert lib.nvtext_amd_fixed_to_arrow_device(C.byref(fixed), stream_of(env), C.byref(env["mr"].struct), C.byref(fs), C.byref(fa)) == capi.SUCCESS
    got, keep = import_result(env, fs, fa)
    exp = orc.jaccard_index(host_strings(a1), host_strings(a2), 3)
    assert got.type == pa.float32() and got.null_count == exp.null_count
    assert got.to_pylist() == exp.to_pylist()
    fa.array.release(C.byref(fa.array))


def test_normalize_characters_through_arrow(env):
    capi, lib = env["capi"], env["lib"]
    from oracle import normalize_py
    rows = ["Stock^ $1", None, "éâîô\teaio", "[PAD] ĂĆĖÑÜ", "", "丏丟"]
    normalizer = C.c_void_p()
    tokens = env["nv"].DeviceStringsColumn.from_host(host_strings(pa.array(["[PAD]"], type=pa.string())))._c()
    assert lib.nvtext_amd_character_normalizer_create(1, C.byref(tokens), stream_of(env), C.byref(env["mr"].struct), C.byref(normalizer)) == capi.SUCCESS
    for typ, want in ((pa.string(), pa.string()), (pa.large_string(), pa.string())):
        arr = pa.array(rows, type=typ)
        schema = export_schema(env, typ)
        darr = device_array_of(env, arr)
        col = capi.StringsColumn()
        assert lib.nvtext_amd_strings_from_arrow_device(C.byref(schema), C.byref(darr), stream_of(env), C.byref(col)) == capi.SUCCESS
        out = capi.StringsResult()
        assert lib.nvtext_amd_normalize_characters(C.byref(col), normalizer, stream_of(env), C.byref(env["mr"].struct), C.byref(out)) == capi.SUCCESS
        out_schema, out_arr = capi.ArrowSchema(), capi.ArrowDeviceArray()
        assert lib.nvtext_amd_strings_to_arrow_device(C.byref(out), stream_of(env), C.byref(env["mr"].struct), C.byref(out_schema),
                                                      C.byref(out_arr)) == capi.SUCCESS
        assert not out.offsets and not out.chars  # moved out
        got, keep = import_result(env, out_schema, out_arr)
        exp = normalize_py.normalize_characters(host_strings(arr), True, [b"[PAD]"])
        assert got.type == want and got.null_count == 1
        assert [None if v is None else v.encode("utf-8") for v in got.to_pylist()] == exp.to_pylist()
        out_arr.array.release(C.byref(out_arr.array))
    # an empty result still is a well-formed Arrow string array
    empty = capi.StringsResult()
    col = env["nv"].DeviceStringsColumn.from_host(host_strings(pa.array([], type=pa.string())))._c()
    assert lib.nvtext_amd_normalize_characters(C.byref(col), normalizer, stream_of(env), C.byref(env["mr"].struct), C.byref(empty)) == capi.SUCCESS
    out_schema, out_arr = capi.ArrowSchema(), capi.ArrowDeviceArray()
    assert lib.nvtext_amd_strings_to_arrow_device(C.byref(empty), stream_of(env), C.byref(env["mr"].struct), C.byref(out_schema),
                                                  C.byref(out_arr)) == capi.SUCCESS
    got, keep = import_result(env, out_schema, out_arr)
    assert got.type == pa.string() and len(got) == 0
    out_arr.array.release(C.byref(out_arr.array))
    lib.nvtext_amd_character_normalizer_destroy(normalizer)


def test_arrow_argument_checks(env):
    capi, lib = env["capi"], env["lib"]
    arr = pa.array(["a", "b"], type=pa.string())
    schema = export_schema(env, pa.string())
    col = capi.StringsColumn()
    on_cpu = device_array_of(env, arr, device_type=capi.ARROW_DEVICE_CPU)
    assert lib.nvtext_amd_strings_from_arrow_device(C.byref(schema), C.byref(on_cpu), None, C.byref(col)) == capi.INVALID_ARGUMENT
    ints = export_schema(env, pa.int32())
    ok = device_array_of(env, arr)
    assert lib.nvtext_amd_strings_from_arrow_device(C.byref(ints), C.byref(ok), None, C.byref(col)) == capi.INVALID_ARGUMENT
    lcol = capi.ListStringsColumn()
    assert lib.nvtext_amd_list_strings_from_arrow_device(C.byref(schema), C.byref(ok), None, C.byref(lcol)) == capi.INVALID_ARGUMENT
    empty = capi.ListColumn()
    assert lib.nvtext_amd_list_to_arrow_device(C.byref(empty), None, None, C.byref(capi.ArrowSchema()), C.byref(capi.ArrowDeviceArray())) == capi.INVALID_ARGUMENT
