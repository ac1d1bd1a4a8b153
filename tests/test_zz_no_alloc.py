"""The allocation-free CRC-32C entry point (``mlf_crc32c_device_noalloc``) against the allocating one.

Called through the C-ABI (ctypes).  The two must agree bit for bit; the allocation-free variant keeps its scratch in a
fixed device array that every call on the device shares and that keeps the last call's contents, so the comparison is
made on two calls in a row, the second on a smaller input, and once more after an unrelated call in between.
"""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
_FILL = 0xDEADBEEF - (1 << 32)  # as the int32 the output tensors are typed as


def _u32(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint32)


def _noalloc(buf: torch.Tensor, nbytes: int, chunk: int, out: torch.Tensor, stream=None) -> int:
    from ml_flashpoint.hip import _lib

    if stream is None:
        stream = torch.cuda.current_stream(buf.device).cuda_stream
    return _lib.load().mlf_crc32c_device_noalloc(buf.data_ptr(), nbytes, chunk, out.data_ptr(), out.numel(), stream)


def _random_bytes(n: int, seed: int) -> torch.Tensor:
    gen = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randint(0, 256, (n,), dtype=torch.uint8, device=DEV, generator=gen)


def test_noalloc_crc_matches_the_allocating_entry_point_on_two_calls_in_a_row(oracle_c):
    from ml_flashpoint.hip import _lib
    from ml_flashpoint.hip import plan as P

    big_n, small_n = (96 << 20) + 12345, (5 << 20) + 77
    chunk_big, chunk_small = 4 << 20, 1 << 20
    big, small = _random_bytes(big_n, 1), _random_bytes(small_n, 2)
    want_big = P.crc32c_device(big, big_n, chunk_big)
    want_small = P.crc32c_device(small, small_n, chunk_small)
    # the oracle's routine on the small input pins the reference values themselves
    raw = small.cpu().numpy().tobytes()
    oracle = np.zeros(len(want_small), dtype=np.uint32)
    oracle_c.oracle_crc32c_chunks(raw, small_n, chunk_small, oracle.ctypes.data)
    assert want_small.tolist() == oracle.tolist()

    out_big = torch.full((len(want_big) + 3,), _FILL, dtype=torch.int32, device=DEV)
    out_small = torch.full((len(want_small) + 3,), _FILL, dtype=torch.int32, device=DEV)
    free_before, _ = torch.cuda.mem_get_info()
    # two calls in a row on one stream, the second with the smaller input: it must not see what the first left behind
    _lib.check(_noalloc(big, big_n, chunk_big, out_big), "mlf_crc32c_device_noalloc")
    _lib.check(_noalloc(small, small_n, chunk_small, out_small), "mlf_crc32c_device_noalloc")
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, "the allocation-free entry point changed the device's free memory"
    got_big, got_small = _u32(out_big), _u32(out_small)
    assert got_big[: len(want_big)].tolist() == want_big.tolist()
    assert got_small[: len(want_small)].tolist() == want_small.tolist()
    assert (got_big[len(want_big):] == 0xDEADBEEF).all() and (got_small[len(want_small):] == 0xDEADBEEF).all()
    # and again in the other order, on a side stream, after the allocating entry point ran in between
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    out_small.zero_()
    out_big.zero_()
    torch.cuda.synchronize()
    _lib.check(_noalloc(small, small_n, chunk_small, out_small, side.cuda_stream), "mlf_crc32c_device_noalloc")
    _lib.check(_noalloc(big, big_n, chunk_big, out_big, side.cuda_stream), "mlf_crc32c_device_noalloc")
    side.synchronize()
    assert _u32(out_big)[: len(want_big)].tolist() == want_big.tolist()
    assert _u32(out_small)[: len(want_small)].tolist() == want_small.tolist()


def test_noalloc_crc_known_vectors_and_short_inputs():
    """RFC 3720 B.4 vectors and inputs shorter than one 1 KiB row, one segment, one chunk."""
    from ml_flashpoint.hip import _lib

    cases = [(b"123456789", 0xE3069283), (bytes(32), 0x8A9136AA), (b"\xff" * 32, 0x62A8AB43),
             (bytes(range(32)), 0x46DD794E), (bytes(range(31, -1, -1)), 0x113FDB5C)]
    out = torch.zeros(1, dtype=torch.int32, device=DEV)
    for data, want in cases:
        buf = torch.zeros(64, dtype=torch.uint8, device=DEV)
        buf[: len(data)] = torch.frombuffer(bytearray(data), dtype=torch.uint8).to(DEV)
        _lib.check(_noalloc(buf, len(data), 65536, out), "mlf_crc32c_device_noalloc")
        torch.cuda.synchronize()
        assert int(_u32(out)[0]) == want


def test_noalloc_crc_refuses_what_does_not_fit_and_bad_arguments():
    from ml_flashpoint.hip import _lib

    lib = _lib.load()
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    out = torch.zeros(16, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    # 64 KiB chunks pin the segment size at 64 KiB: 262 145 segments do not fit the fixed array (refused before
    # anything is launched, so the buffer's real size does not matter)
    too_many = 65536 * (256 * 1024 + 1)
    rc = lib.mlf_crc32c_device_noalloc(buf.data_ptr(), too_many, 65536, out.data_ptr(), 1 << 40, stream)
    assert rc != 0 and b"fixed scratch array holds 262144" in lib.mlf_hip_last_error()
    assert lib.mlf_crc32c_device_noalloc(buf.data_ptr(), 1 << 20, 65536, out.data_ptr(), 15, stream) != 0  # 16 chunks
    assert b"output array too small" in lib.mlf_hip_last_error()
    assert lib.mlf_crc32c_device_noalloc(buf.data_ptr(), 1 << 20, 1000, out.data_ptr(), 16, stream) != 0
    assert lib.mlf_crc32c_device_noalloc(buf.data_ptr() + 1, 1 << 19, 65536, out.data_ptr(), 16, stream) != 0
    assert lib.mlf_crc32c_device_noalloc(buf.data_ptr(), 1 << 20, 65536, None, 16, stream) != 0
    assert lib.mlf_crc32c_device_noalloc(buf.data_ptr(), 0, 65536, None, 0, stream) == 0  # nothing to do
    torch.cuda.synchronize()


def test_noalloc_crc_inside_a_captured_graph_replayed_over_changing_data():
    """The entry point enqueues kernels and nothing else, so it may be recorded into a HIP graph - once
    ``mlf_hip_set_device`` (or an earlier call) has resolved where the scratch array lies on the device.  Every replay,
    with other work of the program and synchronizations in between, yields what the allocating entry point yields
    for the data the buffer holds at that moment."""
    from ml_flashpoint.hip import _lib
    from ml_flashpoint.hip import plan as P

    lib = _lib.load()
    _lib.check(lib.mlf_hip_set_device(torch.cuda.current_device()), "mlf_hip_set_device")  # resolves the array's address
    nbytes, chunk = (24 << 20) + 4096, 2 << 20
    n_chunks = -(-nbytes // chunk)
    data = _random_bytes(nbytes, 7)
    out = torch.full((n_chunks + 2,), _FILL, dtype=torch.int32, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    free_before, _ = torch.cuda.mem_get_info()
    with torch.cuda.graph(graph, stream=side):
        rc = lib.mlf_crc32c_device_noalloc(data.data_ptr(), nbytes, chunk, out.data_ptr(), out.numel(),
                                           torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "mlf_crc32c_device_noalloc under capture")
    assert (_u32(out) == 0xDEADBEEF).all(), "capturing must not run anything"
    other = _random_bytes((3 << 20) + 5, 9)
    for replay in range(4):
        if replay:
            data.copy_(_random_bytes(nbytes, 100 + replay))  # the program's own eager work between the replays ...
            P.crc32c_device(other, other.numel(), 1 << 20)    # ... including a call that uses other scratch
        out.fill_(_FILL)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = P.crc32c_device(data, nbytes, chunk)
        got = _u32(out)
        assert got[:n_chunks].tolist() == want.tolist(), f"replay {replay}"
        assert (got[n_chunks:] == 0xDEADBEEF).all()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after >= free_before - (8 << 20)  # the graph object itself is all that was added
