"""nvtext_amd_minhash_preallocated, the entry point that allocates nothing on the device, against nvtext_amd_minhash on
the same inputs: bit-exact, on two calls in a row that share the library's scratch array (the second one smaller)."""
import numpy as np
import pytest

from cudf_amd.arrow_host import HostStringsColumn, pack_validity

pytestmark = pytest.mark.gpu


def _column(rng, rows, long_rows, with_nulls):
    lengths = rng.integers(0, 400, rows)
    lengths[rng.integers(0, rows, long_rows)] = rng.integers(16385, 60000, long_rows)  # rows that take extra workgroups
    offsets = np.zeros(rows + 1, np.int32)
    np.cumsum(lengths, out=offsets[1:])
    chars = rng.integers(97, 123, int(offsets[-1]), dtype=np.uint8)
    chars[rng.random(chars.size) < 0.15] = 32
    if not with_nulls:
        return HostStringsColumn(chars, offsets, None, rows, 0, 0)
    valid = rng.random(rows) > 0.1
    return HostStringsColumn(chars, offsets, pack_validity(valid), rows, 0, int((~valid).sum()))


def _both(nv, torch, host, P, width, seed):
    rng = np.random.default_rng(P)
    a = torch.from_numpy(rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32).view(np.int32)).cuda()
    b = torch.from_numpy(rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32).view(np.int32)).cuda()
    col = nv.DeviceStringsColumn.from_host(host)
    exp = nv.minhash(col, seed, a, b, width).to_host()

    offsets = torch.full((host.size + 1,), -1, dtype=torch.int32, device="cuda")
    child = torch.full(((host.size - host.null_count) * P + 5,), -1, dtype=torch.int32, device="cuda")
    mask = torch.zeros(((host.size + 31) // 32,), dtype=torch.int32, device="cuda") if host.mask is not None else None
    # a call of a few rows first: the one-time lookup of the scratch array's address on this device is not what is checked
    warm = nv.DeviceStringsColumn.from_host(HostStringsColumn.from_pylist(["warm up", "the symbol lookup"]))
    nv.minhash_preallocated(warm, seed, a, b, width, torch.zeros(3, dtype=torch.int32, device="cuda"),
                            torch.zeros(2 * P, dtype=torch.int32, device="cuda"), None)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]   # hipMemGetInfo: sees a plain hipMalloc, which torch's own count does not
    nv.minhash_preallocated(col, seed, a, b, width, offsets, child, mask)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "the call took device memory"
    assert np.array_equal(offsets.cpu().numpy(), exp.offsets)
    got = child.cpu().numpy().view(np.uint32)
    assert np.array_equal(got[:exp.child.size], exp.child)
    assert (got[exp.child.size:] == 0xFFFFFFFF).all()           # nothing written past the result
    if mask is not None:
        words = mask.cpu().numpy().view(np.uint32)
        bits = np.unpackbits(words.view(np.uint8), bitorder="little")[:host.size].astype(bool)
        assert np.array_equal(bits, exp.validity())


def test_minhash_preallocated_matches_minhash_on_two_calls_in_a_row():
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from cudf_amd import _capi, nvtext
    _capi.load()
    rng = np.random.default_rng(77)
    _both(nvtext, torch, _column(rng, 200_000, 40, True), 64, 5, 42)
    _both(nvtext, torch, _column(rng, 3_000, 5, False), 26, 12, 0)   # smaller: the scratch still holds the first call's values
    _both(nvtext, torch, _column(rng, 1, 0, False), 260, 4, 1)


def test_minhash_preallocated_refuses_more_rows_than_its_scratch_holds():
    import torch
    from cudf_amd import _capi, nvtext
    _capi.load()
    rows = nvtext.MINHASH_PREALLOCATED_MAX_ROWS + 1
    host = HostStringsColumn(np.zeros(0, np.uint8), np.zeros(rows + 1, np.int32), None, rows, 0, 0)
    col = nvtext.DeviceStringsColumn.from_host(host)
    a = torch.ones(1, dtype=torch.int32, device="cuda")
    offsets = torch.zeros(rows + 1, dtype=torch.int32, device="cuda")
    child = torch.zeros(rows, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="NVTEXT_AMD_MINHASH_PREALLOCATED_MAX_ROWS"):
        nvtext.minhash_preallocated(col, 0, a, a, 4, offsets, child, None)
    # the largest size it takes
    col = nvtext.DeviceStringsColumn.from_host(HostStringsColumn(np.zeros(0, np.uint8), np.zeros(rows, np.int32), None, rows - 1, 0, 0))
    nvtext.minhash_preallocated(col, 0, a, a, 4, offsets, child, None)
    torch.cuda.synchronize()
    assert int(offsets[rows - 1]) == rows - 1 and int(child.abs().sum()) == 0   # empty rows: zeros


def test_minhash_preallocated_recorded_into_a_hip_graph_and_replayed():
    """What the entry point is for: a caller under HIP graph capture.  The call is recorded once (after a call outside of
    any capture, which looks the scratch array's address up) and replayed on new bytes in the same buffers, with eager work
    and synchronisations of the program's own between the replays; every replay against nvtext_amd_minhash run eagerly."""
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from cudf_amd import _capi, nvtext as nv
    _capi.load()
    rng = np.random.default_rng(99)
    host = _column(rng, 20_000, 6, True)
    P, width, seed = 129, 5, 7
    a = torch.from_numpy(rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32).view(np.int32)).cuda()
    b = torch.from_numpy(rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32).view(np.int32)).cuda()
    col = nv.DeviceStringsColumn.from_host(host)
    offsets = torch.full((host.size + 1,), -1, dtype=torch.int32, device="cuda")
    child = torch.full(((host.size - host.null_count) * P,), -1, dtype=torch.int32, device="cuda")
    mask = torch.zeros(((host.size + 31) // 32,), dtype=torch.int32, device="cuda")
    nv.minhash_preallocated(col, seed, a, b, width, offsets, child, mask)   # outside of capture: the address lookup
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.graph(graph, stream=side):
        nv.minhash_preallocated(col, seed, a, b, width, offsets, child, mask)
    torch.cuda.synchronize()
    for replay in range(4):
        # new bytes in the same buffer (the rows keep their lengths); the results cleared, so that a replay that does nothing shows
        fresh = rng.integers(97, 123, host.chars.size, dtype=np.uint8)
        fresh[rng.random(fresh.size) < 0.15] = 32
        col.chars.copy_(torch.from_numpy(fresh).cuda())
        child.fill_(-1)
        offsets.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        exp = nv.minhash(col, seed, a, b, width).to_host()   # eager, same device bytes
        assert np.array_equal(offsets.cpu().numpy(), exp.offsets), replay
        assert np.array_equal(child.cpu().numpy().view(np.uint32), exp.child), replay
        assert (torch.rand(1000, device="cuda").sum() > 0).item()   # eager work of the program's own between replays
