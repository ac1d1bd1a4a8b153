"""Host buffer layer: native BufferObject, BufferIO, BufferPool, CheckpointObjectManager.

Behaviours are the ones the reference's tests pin (tests/checkpoint_object_manager/test_buffer_io.py,
test_checkpoint_object_manager.py, buffer_object/test_buffer_object_bindings.py, tests/core/test_buffer_pool.py),
re-expressed against this package.
"""

import io
import os
import struct

import pytest

from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE, BufferMetadataType
from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.buffer_pool import BufferPool, BufferPoolConfig, PooledBufferIO
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId


# ---- native object ------------------------------------------------------------------------------------------
def test_create_properties_and_memoryview(tmp_path):
    p = str(tmp_path / "sub" / "dir" / "buf")  # parents are created
    bo = BufferObject(p, capacity=1024, overwrite=False)
    assert bo.get_id() == p and bo.get_capacity() == 1024 and bo.closed is False and bo.is_readonly is False
    mv = memoryview(bo)
    assert mv.nbytes == 1024 and not mv.readonly and mv.format == "B" and mv.ndim == 1
    assert bo.get_data_ptr() != 0
    mv.release()
    bo.close()
    assert bo.closed and bo.get_capacity() == 0
    with pytest.raises(RuntimeError, match="Buffer is closed"):
        bo.get_data_ptr()


def test_overwrite_flag_and_error_text(tmp_path):
    p = str(tmp_path / "x")
    BufferObject(p, capacity=32, overwrite=False).close()
    with pytest.raises(RuntimeError, match="File already exists and overwrite is set to false"):
        BufferObject(p, capacity=32, overwrite=False)
    bo = BufferObject(p, capacity=64, overwrite=True)
    assert bo.get_capacity() == 64
    bo.close()
    with pytest.raises(RuntimeError, match="requires a size greater than 0"):
        BufferObject(str(tmp_path / "zero"), capacity=0, overwrite=True)


def test_write_close_reopen_readonly(tmp_path):
    p = str(tmp_path / "rw")
    bo = BufferObject(p, capacity=128, overwrite=True)
    mv = memoryview(bo)
    mv[:20] = b"Hello, BufferObject!"
    mv.release()
    bo.close()
    ro = BufferObject(p)
    mv = memoryview(ro)
    assert ro.get_capacity() == 128 and ro.is_readonly and mv.readonly and mv[:20].tobytes() == b"Hello, BufferObject!"
    with pytest.raises(TypeError):
        mv[0] = 65
    with pytest.raises(RuntimeError, match="read-only"):
        ro.resize(256)
    mv.release()
    ro.close(truncate_size=10)  # ignored for read-only mappings
    assert os.path.getsize(p) == 128


def test_open_errors(tmp_path):
    with pytest.raises(RuntimeError, match="Path is a directory, not a file"):
        BufferObject(str(tmp_path))
    empty = tmp_path / "empty"
    empty.write_bytes(b"")
    with pytest.raises(RuntimeError, match="File cannot be empty"):
        BufferObject(str(empty))
    with pytest.raises(RuntimeError, match="No such file or directory"):
        BufferObject(str(tmp_path / "missing"))


def test_closed_object_buffer_error_and_idempotent_close(tmp_path):
    bo = BufferObject(str(tmp_path / "c"), capacity=16, overwrite=True)
    bo.close()
    bo.close()
    bo.close()
    with pytest.raises(BufferError) as exc:
        memoryview(bo)
    assert isinstance(exc.value.__cause__, RuntimeError)
    assert "Cannot create buffer view on a closed BufferObject" in str(exc.value.__cause__)
    with pytest.raises(RuntimeError, match="closed buffer"):
        bo.resize(32)


def test_close_truncates_and_resize_keeps_contents(tmp_path):
    p = str(tmp_path / "t")
    bo = BufferObject(p, capacity=8192, overwrite=True)
    mv = memoryview(bo)
    mv[:4] = b"abcd"
    mv.release()
    bo.resize(16384)
    assert bo.get_capacity() == 16384 and os.path.getsize(p) == 16384
    assert memoryview(bo)[:4].tobytes() == b"abcd"
    with pytest.raises(RuntimeError, match="resize buffer to 0"):
        bo.resize(0)
    bo.close(truncate_size=100)
    assert os.path.getsize(p) == 100


# ---- BufferIO -------------------------------------------------------------------------------------------------
@pytest.fixture
def rw(tmp_path):
    stream = BufferIO(BufferObject(str(tmp_path / "io.bin"), METADATA_SIZE + 1024, True))
    yield stream
    stream.close()


def test_data_lands_after_the_metadata_block(rw, tmp_path):
    assert rw.write(b"payload!") == 8
    raw = rw.raw_view()
    assert raw[METADATA_SIZE : METADATA_SIZE + 8].tobytes() == b"payload!"
    assert struct.unpack_from("<Q", raw, 0)[0] == 8
    rw.set_format_signature(b"MLF_TENS")
    assert raw[8:16].tobytes() == b"MLF_TENS" and rw.format_signature == b"MLF_TENS"
    with pytest.raises(ValueError, match="at most 8 bytes"):
        rw.set_format_signature(b"123456789")


def test_high_water_mark_seek_and_read_clamping(rw):
    rw.write(b"0123456789")
    assert rw.tell() == 10 and rw.len_written_data == 10
    rw.seek(2)
    rw.write(b"AB")
    assert rw.len_written_data == 10  # overwrite inside: mark unchanged
    assert rw.seek(0) == 0 and rw.read() == b"01AB456789"
    assert rw.read() == b"" and rw.read(5) == b""
    assert rw.seek(-3, io.SEEK_END) == 7 and rw.read(100) == b"789"
    assert rw.seek(1, io.SEEK_SET) == 1 and rw.seek(2, io.SEEK_CUR) == 3
    rw.seek(50)
    assert rw.read(4) == b""  # beyond the mark
    with pytest.raises(ValueError, match="invalid whence"):
        rw.seek(0, 9)
    with pytest.raises(ValueError, match="Negative seek position"):
        rw.seek(-1)
    assert rw.write(b"") == 0


def test_readinto(rw):
    rw.write(b"abcdefgh")
    rw.seek(2)
    target = bytearray(4)
    assert rw.readinto(target) == 4 and bytes(target) == b"cdef"
    big = bytearray(10)
    assert rw.readinto(big) == 2 and bytes(big[:2]) == b"gh"
    assert rw.readinto(bytearray(3)) == 0 and rw.readinto(bytearray(0)) == 0
    with pytest.raises(TypeError, match="writable bytes-like"):
        rw.readinto(b"immutable")
    with pytest.raises(TypeError):
        rw.readinto(memoryview(b"ro"))


def test_capacity_is_enforced(rw):
    with pytest.raises(ValueError, match="exceeds buffer capacity"):
        rw.write(b"x" * 1025)
    rw.write(b"x" * 1000)
    with pytest.raises(ValueError, match="exceeds buffer capacity"):
        rw.next_buffer_slice(25)
    with pytest.raises(ValueError, match="non-negative"):
        rw.next_buffer_slice(-1)
    view = rw.next_buffer_slice(24)
    view[:] = b"y" * 24
    view.release()
    assert rw.tell() == 1024 and rw.len_written_data == 1024
    assert rw.data_address(4) == rw.buffer_obj.get_data_ptr() + METADATA_SIZE + 4


def test_close_truncates_file_to_written_size(tmp_path):
    p = str(tmp_path / "trunc.bin")
    stream = BufferIO(BufferObject(p, METADATA_SIZE + 4096, True))
    stream.write(b"z" * 123)
    stream.close()
    assert os.path.getsize(p) == METADATA_SIZE + 123
    assert stream.closed
    stream.close()  # idempotent
    with pytest.raises(ValueError, match="closed BufferIO"):
        stream.tell()
    keep = BufferIO(BufferObject(str(tmp_path / "keep.bin"), METADATA_SIZE + 4096, True))
    keep.write(b"q")
    keep.close(truncate=False)
    assert os.path.getsize(str(tmp_path / "keep.bin")) == METADATA_SIZE + 4096


def test_readonly_stream(tmp_path):
    p = str(tmp_path / "ro.bin")
    with BufferIO(BufferObject(p, METADATA_SIZE + 64, True)) as w:
        w.set_format_signature(b"TORCH___")
        w.write(b"readonly-data")
    with BufferIO(BufferObject(p)) as r:
        assert r.is_readonly and r.format_signature == b"TORCH___" and r.read() == b"readonly-data"
        for op, args in (("write", (b"x",)), ("next_buffer_slice", (1,)), ("set_format_signature", (b"A",)), ("resize", (8192,))):
            with pytest.raises(TypeError, match="not supported in read-only mode"):
                getattr(r, op)(*args)
    assert os.path.getsize(p) == METADATA_SIZE + 13  # a read-only close never truncates


def test_resize_keeps_the_whole_metadata_block(tmp_path):
    stream = BufferIO(BufferObject(str(tmp_path / "rs.bin"), METADATA_SIZE + 100, True))
    stream.set_format_signature(b"MLF_TENS")
    stream.write(b"k" * 100)
    before = stream.raw_view()[:METADATA_SIZE].tobytes()
    stream.resize(METADATA_SIZE + 100000)
    assert stream.raw_view()[:METADATA_SIZE].tobytes() == before
    stream.write(b"m" * 50000)  # the live metadata view follows the new mapping
    assert stream.len_written_data == 50100
    with pytest.raises(ValueError, match="at least 4096"):
        stream.resize(100)
    stream.close()


def test_constructor_validation(tmp_path):
    closed = BufferObject(str(tmp_path / "c.bin"), 8192, True)
    closed.close()
    with pytest.raises(ValueError, match="closed BufferObject"):
        BufferIO(closed)
    with pytest.raises(ValueError, match="at least 4096"):
        BufferIO(BufferObject(str(tmp_path / "small.bin"), 100, True))
    assert BufferMetadataType.len_written_data.offset == 0 and BufferMetadataType.format_signature.offset == 8


# ---- pool -------------------------------------------------------------------------------------------------------
def test_pool_preallocates_named_files_and_links(tmp_path):
    pool = BufferPool(str(tmp_path / "pool"), rank=3, num_buffers=2, buffer_size=METADATA_SIZE + 1000)
    names = sorted(os.listdir(tmp_path / "pool"))
    assert names == ["buffer_3_0.dist", "buffer_3_1.dist"]
    assert all(os.path.getsize(tmp_path / "pool" / n) == METADATA_SIZE + 1000 for n in names)
    link = str(tmp_path / "obj_a.distcp")
    buf = pool.acquire(link)
    assert isinstance(buf, PooledBufferIO) and os.path.islink(link)
    assert os.path.dirname(os.readlink(link)) == str(tmp_path / "pool")
    buf.write(b"hello")
    buf.close()
    assert buf.closed and os.path.getsize(link) == METADATA_SIZE + 5  # truncated, mapping kept by the pool
    pool.acquire(str(tmp_path / "obj_b.distcp"))
    with pytest.raises(RuntimeError, match="BufferPool exhausted. All 2 buffers are in use."):
        pool.acquire(str(tmp_path / "obj_c.distcp"))
    os.remove(link)  # deleting the checkpoint object frees its buffer
    again = pool.acquire(str(tmp_path / "obj_c.distcp"))
    assert again.tell() == 0 and again.len_written_data == 0
    pool.teardown()


def test_pool_auto_resize_formula(tmp_path):
    pool = BufferPool(str(tmp_path / "pool"), num_buffers=1, buffer_size=METADATA_SIZE + 100)
    buf = pool.acquire(str(tmp_path / "o.distcp"))
    buf.write(b"a" * 100)  # fits exactly: no growth
    assert buf.buffer_obj.get_capacity() == METADATA_SIZE + 100
    buf.write(b"b" * 10)
    expected = int(max((METADATA_SIZE + 100) * 1.1, METADATA_SIZE + 100 + 10 + 1024 * 1024))
    assert buf.buffer_obj.get_capacity() == expected
    view = buf.next_buffer_slice(3 * 1024 * 1024)
    view.release()
    assert buf.buffer_obj.get_capacity() >= METADATA_SIZE + 110 + 3 * 1024 * 1024
    buf.seek(0)
    assert buf.read(105) == b"a" * 100 + b"b" * 5
    buf.close()
    pool.teardown()


def test_pool_symlink_failure_returns_buffer(tmp_path):
    pool = BufferPool(str(tmp_path / "pool"), num_buffers=1, buffer_size=METADATA_SIZE + 10)
    with pytest.raises(OSError):
        pool.acquire(str(tmp_path / "no_such_dir" / "o.distcp"))
    assert len(pool.free_buffers) == 1 and not pool.active_buffers
    pool.teardown()
    with pytest.raises(ValueError):
        BufferPool("", num_buffers=1, buffer_size=10)
    with pytest.raises(ValueError):
        BufferPool(str(tmp_path), num_buffers=0, buffer_size=10)
    with pytest.raises(ValueError):
        BufferPoolConfig(str(tmp_path), rank=-1, num_buffers=1, buffer_size=1)


# ---- manager ----------------------------------------------------------------------------------------------------
@pytest.fixture
def no_pool():
    CheckpointObjectManager._worker_pool = None
    yield
    CheckpointObjectManager().teardown_pool()


def test_manager_acquire_adds_metadata_block_and_overwrites(tmp_path, no_pool):
    mgr = CheckpointObjectManager()
    oid = CheckpointObjectId(str(tmp_path / "step-1_ckpt" / "o.distcp"))
    with mgr.acquire_buffer(oid, 1000) as w:
        assert w.buffer_obj.get_capacity() == 1000 + METADATA_SIZE
        w.write(b"first")
    with pytest.raises(FileExistsError):
        mgr.acquire_buffer(oid, 1000, overwrite=False)
    with mgr.acquire_buffer(oid, 10) as w:  # default: overwrite
        w.write(b"second")
    with mgr.get_buffer(oid) as r:
        assert r.read() == b"second"
    with pytest.raises(ValueError, match="positive integer"):
        mgr.acquire_buffer(oid, 0)
    assert mgr.get_buffer(CheckpointObjectId(str(tmp_path / "absent"))) is None
    assert mgr.get_buffer(CheckpointObjectId(str(tmp_path / "step-1_ckpt"))) is None  # a directory
    mgr.delete_object(oid)
    assert not os.path.exists(str(oid))
    mgr.delete_container(CheckpointContainerId(str(tmp_path / "step-1_ckpt")))
    assert not os.path.exists(str(tmp_path / "step-1_ckpt"))


def test_manager_prefers_pool_then_falls_back(tmp_path, no_pool):
    mgr = CheckpointObjectManager(BufferPoolConfig(str(tmp_path / "pool"), 0, 1, METADATA_SIZE + 64))
    a = CheckpointObjectId(str(tmp_path / "ck" / "a.distcp"))
    b = CheckpointObjectId(str(tmp_path / "ck" / "b.distcp"))
    wa = mgr.acquire_buffer(a, 64)
    assert isinstance(wa, PooledBufferIO) and os.path.islink(str(a))
    wb = mgr.acquire_buffer(b, 64)  # pool exhausted: standalone file
    assert isinstance(wb, BufferIO) and not os.path.islink(str(b))
    wa.close()
    wb.close()
    mgr.close_buffer(wb)  # closing a closed buffer is ignored
    # another manager in the same process shares the pool
    assert CheckpointObjectManager()._get_or_create_buffer_pool() is CheckpointObjectManager._worker_pool


def test_a_buffer_is_never_made_larger_than_its_file_system_can_hold(shm_dir):
    """Stores into pages a full tmpfs cannot back end in SIGBUS, so creation and growth beyond the free space are
    refused with an error instead (the file is sparse: asking costs nothing)."""
    free = os.statvfs(shm_dir)
    too_much = free.f_bavail * free.f_frsize + (1 << 30)
    path = os.path.join(shm_dir, "too_large.bin")
    with pytest.raises(RuntimeError, match="not enough space on the file system"):
        BufferObject(path, capacity=too_much, overwrite=True)
    assert not os.path.exists(path)                                # nothing is left behind
    bo = BufferObject(path, capacity=METADATA_SIZE + 100, overwrite=True)
    memoryview(bo)[:3] = b"abc"
    with pytest.raises(RuntimeError, match="not enough space on the file system"):
        bo.resize(too_much)
    assert not bo.closed and bo.get_capacity() == METADATA_SIZE + 100  # refused growth leaves the buffer as it was
    assert bytes(memoryview(bo)[:3]) == b"abc"
    bo.resize(METADATA_SIZE + 200)
    bo.close()


def test_reserve_allocates_the_pages_of_a_range_ahead_of_the_writer(shm_dir):
    path = os.path.join(shm_dir, "reserve.bin")
    bo = BufferObject(path, capacity=METADATA_SIZE + (8 << 20), overwrite=True)
    assert os.stat(path).st_blocks * 512 < (1 << 20)             # sparse: nothing allocated yet
    bo.reserve(offset=METADATA_SIZE, nbytes=4 << 20)
    allocated = os.stat(path).st_blocks * 512
    assert (4 << 20) <= allocated < (6 << 20)                     # that range and nothing like the whole file
    assert bytes(memoryview(bo)[METADATA_SIZE : METADATA_SIZE + 16]) == bytes(16)   # reserved pages read as zeros
    bo.reserve(METADATA_SIZE, 4 << 20)                            # already there: nothing to do
    assert os.stat(path).st_blocks * 512 == allocated
    with pytest.raises(RuntimeError, match="outside the buffer"):
        bo.reserve(METADATA_SIZE, 9 << 20)
    stream = BufferIO(bo)
    stream.write(b"x" * 100)
    stream.reserve(6 << 20)                                       # from the current position on
    assert os.stat(path).st_blocks * 512 >= METADATA_SIZE + 100 + (6 << 20) - 4096
    stream.close()
    ro = BufferIO(BufferObject(path))
    with pytest.raises(TypeError, match="read-only"):
        ro.reserve(10)
    with pytest.raises(RuntimeError, match="read-only"):
        ro.buffer_obj.reserve(0, 10)
    ro.close()


def test_pool_prefaults_its_files_in_the_background(shm_dir):
    """A pool of files large enough to be worth it allocates and maps their pages on a background thread; a buffer
    is lent out only once its own file is done, holds what is written into it, and shrinks to the exact size."""
    import os

    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.core.buffer_pool import BufferPool, BufferPoolConfig
    from ml_flashpoint.core.checkpoint_id_types import CheckpointObjectId

    size = 96 << 20
    pool = BufferPool(os.path.join(shm_dir, "pool"), rank=3, num_buffers=2, buffer_size=size, prefault=True)
    assert pool._prefault_worker is not None
    stream = pool.acquire(os.path.join(shm_dir, "object.distcp"))  # waits for the file it gets
    path = stream.buffer_obj.get_id()
    assert os.stat(path).st_blocks * 512 >= size, "the file's pages were not allocated ahead of the writer"
    payload = bytes(range(256)) * 4096
    stream.write(payload)
    stream.close()
    assert os.path.getsize(path) == METADATA_SIZE + len(payload)
    assert open(os.path.join(shm_dir, "object.distcp"), "rb").read()[METADATA_SIZE:] == payload
    assert pool.wait_prefault() > 0.0
    other = [p for p in os.listdir(os.path.join(shm_dir, "pool")) if not path.endswith(p)]
    assert len(other) == 1 and os.stat(os.path.join(shm_dir, "pool", other[0])).st_blocks * 512 >= size
    pool.teardown()
    # small files, or prefault=False: no thread, pages left to the first write as in the reference
    assert BufferPool(os.path.join(shm_dir, "small"), num_buffers=1, buffer_size=1 << 20, prefault=True)._prefault_worker is None
    lazy = BufferPool(os.path.join(shm_dir, "lazy"), num_buffers=1, buffer_size=size)
    assert lazy._prefault_worker is None and os.stat(lazy.free_buffers[0].buffer_obj.get_id()).st_blocks * 512 < size
    lazy.teardown()
    # through the manager: the pool can be created, and waited for, before the first save
    CheckpointObjectManager._worker_pool = None
    manager = CheckpointObjectManager(BufferPoolConfig(os.path.join(shm_dir, "managed"), 0, 1, size, prefault=True))
    assert manager.warm_up_pool(wait=True) > 0.0
    with manager.acquire_buffer(CheckpointObjectId(os.path.join(shm_dir, "ckpt", "a.distcp")), 1 << 20) as writer:
        writer.write(b"abc")
    assert open(os.path.join(shm_dir, "ckpt", "a.distcp"), "rb").read()[METADATA_SIZE:] == b"abc"
    manager.teardown_pool()
    assert CheckpointObjectManager(None).warm_up_pool() == 0.0
    # the default is the reference's: sparse pool files, nothing committed before a save writes it
    assert BufferPoolConfig(os.path.join(shm_dir, "sparse"), 0, 1, size).prefault is False
    manager = CheckpointObjectManager(BufferPoolConfig(os.path.join(shm_dir, "sparse"), 0, 1, size))
    assert manager.warm_up_pool(wait=True) == 0.0
    pool_file = os.path.join(shm_dir, "sparse", "buffer_0_0.dist")
    assert os.path.getsize(pool_file) == size and os.stat(pool_file).st_blocks * 512 < size
    manager.teardown_pool()


def test_pool_prefault_is_skipped_when_memory_is_short(shm_dir, monkeypatch):
    """Prefaulting commits the whole pool; with less than that to spare (file system or host) it does not start."""
    import logging
    import os

    from ml_flashpoint.core import buffer_pool

    monkeypatch.setattr(buffer_pool, "_spare_bytes", lambda directory: 100 << 20)
    size = 96 << 20
    seen = []
    handler = logging.Handler()
    handler.emit = lambda record: seen.append(record.getMessage())
    buffer_pool._LOGGER.addHandler(handler)
    try:
        pool = buffer_pool.BufferPool(os.path.join(shm_dir, "tight"), num_buffers=2, buffer_size=size, prefault=True)
    finally:
        buffer_pool._LOGGER.removeHandler(handler)
    assert pool._prefault_worker is None and any("not prefaulting" in m for m in seen)
    path = pool.free_buffers[0].buffer_obj.get_id()
    assert os.stat(path).st_blocks * 512 < size
    with pool.acquire(os.path.join(shm_dir, "o.distcp")) as stream:  # still usable, pages on demand
        stream.write(b"x" * 1000)
    pool.teardown()
    monkeypatch.undo()
    spare = buffer_pool._spare_bytes(shm_dir)
    stat = os.statvfs(shm_dir)
    assert 0 < spare <= stat.f_bavail * stat.f_frsize


def test_pool_waits_for_a_prefault_outside_its_lock(shm_dir):
    """While one acquire waits for its file's pages, the pool's lock is free: another acquire gets the other buffer."""
    import os
    import threading

    from ml_flashpoint.core.buffer_pool import BufferPool

    pool = BufferPool(os.path.join(shm_dir, "pool"), num_buffers=2, buffer_size=1 << 20)
    slow = pool.free_buffers[-1].buffer_obj.get_id()  # the buffer the next acquire takes
    pool._prefaulted[slow] = threading.Event()        # as if its pages were still being mapped
    got = {}
    first = threading.Thread(target=lambda: got.setdefault("first", pool.acquire(os.path.join(shm_dir, "a.distcp"))))
    first.start()
    while slow not in pool.active_buffers:  # taken, and now waiting
        pass
    second = pool.acquire(os.path.join(shm_dir, "b.distcp"))  # would deadlock if the wait held the lock
    assert second.buffer_obj.get_id() != slow and "first" not in got
    with __import__("pytest").raises(RuntimeError, match="exhausted"):
        pool.acquire(os.path.join(shm_dir, "c.distcp"))
    pool._prefaulted[slow].set()
    first.join(5)
    assert got["first"].buffer_obj.get_id() == slow and os.path.islink(os.path.join(shm_dir, "a.distcp"))
    pool.teardown()
