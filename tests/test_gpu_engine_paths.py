"""The copy engine's failure paths and its event-gated transfer, through the C-ABI.

Failures are forced from the host side only (a descriptor that cannot be written, a file shorter than the range asked
for): every kernel and copy that was enqueued still completes normally.  After a failed transfer the engine must say
what went wrong, must not have lost a slot, and must carry out the next transfer correctly.
"""

import ctypes
import os
import time

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _random(nbytes, seed):
    gen = torch.Generator().manual_seed(seed)
    host = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=gen)
    return host, host.to(DEV)


def test_failed_transfers_report_and_leave_the_engine_usable(shm_dir):
    from ml_flashpoint.hip import _lib
    from ml_flashpoint.hip import plan as P

    nbytes = (7 << 20) + 123  # eight slots' worth through a ring of three: slots are reused within one transfer
    host, dev = _random(nbytes, 1)
    engine = P.CopyEngine(slot_bytes=1 << 20, n_slots=3, n_threads=4)
    stream = torch.cuda.current_stream().cuda_stream
    path = os.path.join(shm_dir, "object.bin")
    with open(path, "wb") as f:
        f.truncate(4096 + nbytes)

    for attempt in range(3):  # more failures than the ring has slots: a leaked slot would stall the next transfer
        # device -> file through a descriptor that was opened for reading: pwrite() fails with EBADF
        fd = os.open(path, os.O_RDONLY)
        try:
            with pytest.raises(_lib.HipError, match=r"pwrite\(\) to the buffer file failed: Bad file descriptor"):
                engine.d2h_fd(dev.data_ptr(), fd, 4096, nbytes, stream)
        finally:
            os.close(fd)
        # file -> device past the end of the file: pread() returns 0 bytes, reported as ENODATA
        back = torch.zeros(nbytes + 4096, dtype=torch.uint8, device=DEV)
        fd = os.open(path, os.O_RDONLY)
        try:
            with pytest.raises(_lib.HipError, match=r"pread\(\) from the buffer file failed: No data available"):
                engine.h2d_fd(fd, 4096, back.data_ptr(), nbytes + 4096, stream)
        finally:
            os.close(fd)
        # a closed descriptor
        with pytest.raises(_lib.HipError, match=r"pwrite\(\) to the buffer file failed"):
            engine.d2h_fd(dev.data_ptr(), fd, 4096, nbytes, stream)
        # null pointers and a bad descriptor are refused before anything is enqueued
        lib = _lib.load()
        stats = _lib.XferStats()
        assert lib.mlf_engine_d2h(engine._handle, None, None, 16, stream, ctypes.byref(stats)) != 0
        assert lib.mlf_engine_d2h_fd(engine._handle, dev.data_ptr(), -1, 0, 16, stream, ctypes.byref(stats)) != 0
        assert b"bad file descriptor" in lib.mlf_hip_last_error()

        # the engine still works: the same object through the descriptor and back, with checksums beside the copies
        fd = os.open(path, os.O_RDWR)
        try:
            stats = engine.d2h_fd(dev.data_ptr(), fd, 4096, nbytes, stream)
            assert stats.bytes == nbytes and stats.chunks == 8
            assert os.pread(fd, nbytes, 4096) == host.numpy().tobytes()
            back.zero_()
            engine.h2d_fd(fd, 4096, back.data_ptr(), nbytes, stream)
            torch.cuda.synchronize()
            assert torch.equal(back[:nbytes].cpu(), host) and int(back[nbytes:].sum()) == 0
        finally:
            os.close(fd)
        arena = torch.zeros(nbytes, dtype=torch.uint8)
        _, crcs = engine.d2h_crc(dev.data_ptr(), arena.data_ptr(), nbytes, stream, 1 << 20)
        assert torch.equal(arena, host)
        want = [P.crc32c_host(host.data_ptr() + k * (1 << 20), min(1 << 20, nbytes - k * (1 << 20))) for k in range(8)]
        assert crcs.tolist() == want, attempt
    engine.destroy()


def test_gated_transfer_waits_for_its_event_and_not_for_the_stream():
    """A transfer gated on the event behind its producer starts while later work still occupies the producer's stream;
    the stream-gated form of the same transfer waits for that work.  Same bytes and checksums either way."""
    from ml_flashpoint.hip import plan as P

    nbytes = (3 << 20) + 17
    host, dev = _random(nbytes, 2)
    engine = P.CopyEngine(slot_bytes=1 << 20, n_slots=3, n_threads=4)
    cur = torch.cuda.current_stream()
    landed = ctypes.c_uint64(0)
    arena = torch.zeros(nbytes, dtype=torch.uint8).pin_memory()
    # warm both paths up (first use allocates the checksum scratch)
    ready = torch.cuda.Event()
    ready.record()
    engine.d2h_gated(dev.data_ptr(), arena.data_ptr(), nbytes, ready.cuda_event, 1 << 20, landed)
    engine.d2h_watched(dev.data_ptr(), arena.data_ptr(), nbytes, cur.cuda_stream, 1 << 20, landed)
    torch.cuda.synchronize()

    ballast = torch.zeros(2 << 30, dtype=torch.uint8, device=DEV)

    def busy(seconds):  # occupies the current stream with about that much independent work (~1 ms per pass)
        for _ in range(int(seconds * 1000)):
            ballast.add_(1)

    dev2 = dev.clone()  # "the pack": the producer of what is about to be sent
    ready = torch.cuda.Event()
    ready.record()
    busy(0.6)
    arena.zero_()
    stats, crcs = engine.d2h_gated(dev2.data_ptr(), arena.data_ptr(), nbytes, ready.cuda_event, 1 << 20, landed)
    still_busy = not cur.query()  # asked right behind the transfer: the later work is still on the stream
    assert torch.equal(arena, host) and int(landed.value) == nbytes
    want = [P.crc32c_host(host.data_ptr() + k * (1 << 20), min(1 << 20, nbytes - k * (1 << 20))) for k in range(4)]
    assert crcs.tolist() == want
    torch.cuda.synchronize()

    busy(0.6)
    arena.zero_()
    stats2, crcs2 = engine.d2h_watched(dev2.data_ptr(), arena.data_ptr(), nbytes, cur.cuda_stream, 1 << 20, landed)
    drained = cur.query()  # the stream-gated form can only have started once the stream had run dry
    assert torch.equal(arena, host) and crcs2.tolist() == want
    torch.cuda.synchronize()
    print(f"transfer of {nbytes} bytes behind 0.6 s of later work on the producer's stream: gated on the event "
          f"{stats.seconds * 1e3:.1f} ms (of which waiting {stats.wait_seconds * 1e3:.1f}), gated on the stream "
          f"{stats2.seconds * 1e3:.1f} ms (of which waiting {stats2.wait_seconds * 1e3:.1f})")
    # order, not durations: the event-gated transfer was complete while the later work was still running, the
    # stream-gated one only after it; and the latter spent longer waiting for its gate than the former
    assert still_busy, "the later work had already finished when the event-gated transfer returned"
    assert drained, "the stream-gated transfer returned before the stream had finished its earlier work"
    assert stats2.wait_seconds > stats.wait_seconds
    # no event at all: starts at once
    engine.d2h_gated(dev2.data_ptr(), arena.data_ptr(), nbytes, None, 0, landed)
    assert torch.equal(arena, host)
    engine.destroy()


def test_engines_keep_their_streams_off_the_hardware_queue_of_the_training_stream():
    """HIP spreads a process's streams over a few hardware queues; a copy stream that shares its queue with a stream
    that is kept full crawls.  Several engines are created (so that some of their streams land on the default
    stream's queue), each is told to avoid the default stream, and each must then move data at a sane rate while
    kernels are queued back to back on the default stream - without the call at least one of them would not."""
    import threading

    from ml_flashpoint.hip import plan as P

    n = 2 << 30
    buf = torch.zeros(n, dtype=torch.uint8, device=DEV)
    a = torch.randn(4096, 4096, device=DEV, dtype=torch.bfloat16)
    stop = threading.Event()

    def busy():  # kernels back to back on the default stream, ~10 ms queued at any time
        while not stop.is_set():
            for _ in range(40):
                torch.matmul(a, a)
            torch.cuda.synchronize()

    engines = [P.CopyEngine(slot_bytes=8 << 20, n_slots=3, n_threads=4) for _ in range(5)]

    def rates_beside_a_busy_default_stream():
        stop.clear()
        worker = threading.Thread(target=busy)
        worker.start()
        try:
            time.sleep(0.1)
            return [n / engine.link_probe(buf.data_ptr(), n, True) for engine in engines]
        finally:
            stop.set()
            worker.join()

    try:
        idle = n / engines[0].link_probe(buf.data_ptr(), n, True)
        before = rates_beside_a_busy_default_stream()
        left = [engine.avoid_stream(torch.cuda.current_stream().cuda_stream) for engine in engines]
        assert left == [0] * len(engines)
        rates = rates_beside_a_busy_default_stream()
        print(f"link rate idle {idle / 1e9:.1f} GB/s; beside a busy default stream, as created: "
              + ", ".join(f"{r / 1e9:.1f}" for r in before) + " GB/s; after avoid_stream: "
              + ", ".join(f"{r / 1e9:.1f}" for r in rates) + " GB/s")
        # One engine against the others in the same run, not against a figure: an engine with a stream left on the
        # busy stream's hardware queue moves a quarter of what the others move (measured: 12.7 against 52-53 GB/s).
        assert min(rates) > 0.5 * max(rates), (idle, before, rates)
        assert all(engine.checksum_stream for engine in engines)
    finally:
        for engine in engines:
            engine.destroy()
