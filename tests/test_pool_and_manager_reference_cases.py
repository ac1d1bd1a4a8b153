"""Buffer pool and checkpoint object manager, case by case as the reference's own suites state them
(tests/core/test_buffer_pool.py:25-288, tests/checkpoint_object_manager/test_checkpoint_object_manager.py:102-1035),
restated against real files; where the reference patches a collaborator, a small stand-in class takes its place."""

import os
import pickle

import pytest

from ml_flashpoint.checkpoint_object_manager import checkpoint_object_manager as com_module
from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.buffer_pool import BufferPool, BufferPoolConfig, PooledBufferIO
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId


@pytest.fixture
def pool(tmp_path):
    p = BufferPool(pool_dir_path=str(tmp_path / ".buffer_pool"), rank=0, num_buffers=3, buffer_size=METADATA_SIZE + 1024)
    yield p
    p.teardown()


@pytest.fixture
def manager():
    CheckpointObjectManager._worker_pool = None
    yield CheckpointObjectManager()
    CheckpointObjectManager().teardown_pool()
    CheckpointObjectManager._worker_pool = None


# ---- pool (test_buffer_pool.py:43-126) --------------------------------------------------------------------------------
def test_acquire_hands_out_a_preallocated_buffer(pool):
    buf = pool.acquire()
    assert isinstance(buf, PooledBufferIO)
    buffer_id = buf.buffer_obj.get_id()
    assert "buffer_0_" in buffer_id and os.path.exists(buffer_id)
    assert len(pool.free_buffers) == 2 and len(pool.active_buffers) == 1 and buffer_id in pool.active_buffers
    buf.close()
    assert buf.closed and not buf._buffer_io.closed            # the proxy closes, the pool keeps the mapping


def test_gc_frees_only_buffers_whose_link_is_gone(pool, tmp_path):
    link = str(tmp_path / "my_symlink")
    buf = pool.acquire(associated_symlink=None)
    buffer_id = buf.buffer_obj.get_id()
    assert pool.active_buffers[buffer_id][1] is None
    pool._gc()
    assert buffer_id in pool.active_buffers                     # no link registered yet: not collectable
    buf.close()
    buf = pool.acquire(associated_symlink=link)
    buffer_id = buf.buffer_obj.get_id()
    assert os.path.islink(link) and pool.active_buffers[buffer_id][1] == link
    pool._gc()
    assert buffer_id in pool.active_buffers                     # link alive: stays
    os.remove(link)
    pool._gc()
    assert buffer_id not in pool.active_buffers and buf._buffer_io in pool.free_buffers


def test_failed_link_creation_returns_the_buffer(pool, tmp_path):
    target = str(tmp_path / "symlink_fail")
    os.makedirs(target)                                         # a directory sits where the link should go
    with pytest.raises(OSError):
        pool.acquire(associated_symlink=target)
    assert len(pool.free_buffers) == 3 and len(pool.active_buffers) == 0


def test_pool_and_config_argument_checks():
    with pytest.raises(ValueError, match="Number of buffers must be positive"):
        BufferPool(pool_dir_path="/tmp", num_buffers=0, buffer_size=1024)
    with pytest.raises(ValueError, match="Buffer size must be positive"):
        BufferPool(pool_dir_path="/tmp", num_buffers=3, buffer_size=0)
    with pytest.raises(ValueError, match="Pool directory path must be provided"):
        BufferPool(pool_dir_path="", num_buffers=3, buffer_size=1024)
    cfg = BufferPoolConfig(pool_dir_path="/tmp/pool", rank=0, num_buffers=3, buffer_size=1024)
    assert (cfg.pool_dir_path, cfg.rank, cfg.num_buffers, cfg.buffer_size) == ("/tmp/pool", 0, 3, 1024)
    with pytest.raises(ValueError, match="pool_dir_path must be provided"):
        BufferPoolConfig(pool_dir_path="", rank=0, num_buffers=3, buffer_size=1024)
    good = dict(pool_dir_path="/tmp/pool", rank=0, num_buffers=3, buffer_size=1024)
    for field, bad in (("rank", -1), ("rank", "0"), ("num_buffers", -1), ("num_buffers", "3"),
                       ("buffer_size", -100), ("buffer_size", "1024")):
        with pytest.raises(ValueError, match=f"{field} must be a non-negative integer"):
            BufferPoolConfig(**{**good, field: bad})


# ---- pooled stream (test_buffer_pool.py:129-237) ---------------------------------------------------------------------
class _RecordingStream:
    """What the proxy needs from a BufferIO, recording the calls it receives."""

    class _Obj:
        def __init__(self, capacity):
            self.capacity = capacity

        def get_capacity(self):
            return self.capacity

    class _Meta:
        len_written_data = 500

    def __init__(self, capacity=1000, pos=0):
        self.buffer_obj = self._Obj(capacity)
        self.closed = False
        self.is_readonly = False
        self._metadata = self._Meta()
        self._mv = range(capacity)
        self.pos = pos
        self.calls = []

    def tell(self):
        self.calls.append(("tell",))
        return self.pos

    def resize(self, n):
        self.calls.append(("resize", n))
        self.buffer_obj.capacity = n

    def __getattr__(self, name):
        def record(*args):
            self.calls.append((name, *args))
            return None

        return record

    def named(self, name):
        return [c for c in self.calls if c[0] == name]


def test_proxy_delegates_and_mirrors_state():
    inner = _RecordingStream(capacity=METADATA_SIZE + 1000)
    proxy = PooledBufferIO(inner)
    proxy.read(10)
    proxy.seek(5, 1)
    proxy.flush()
    assert ("read", 10) in inner.calls and ("seek", 5, 1) in inner.calls and ("flush",) in inner.calls
    assert proxy.buffer_obj is inner.buffer_obj and not proxy.closed
    inner.closed = True
    assert proxy.closed
    inner.closed = False
    proxy.write(b"test")                                        # fits: passed on, nothing resized
    proxy.next_buffer_slice(100)
    assert inner.named("write") == [("write", b"test")] and inner.named("next_buffer_slice") == [("next_buffer_slice", 100)]
    assert not inner.named("resize")


def test_proxy_grows_before_a_write_that_does_not_fit():
    inner = _RecordingStream(capacity=1000, pos=0)
    data = b"x" * 1500
    PooledBufferIO(inner).write(data)
    assert inner.named("resize") == [("resize", int(max(1000 * 1.1, METADATA_SIZE + 0 + 1500 + 1024 * 1024)))]
    assert inner.named("write") == [("write", data)]            # once, after the growth
    inner = _RecordingStream(capacity=1000, pos=900)
    PooledBufferIO(inner).next_buffer_slice(200)
    assert len(inner.named("resize")) == 1 and inner.named("next_buffer_slice") == [("next_buffer_slice", 200)]


def test_proxy_close_truncates_the_file_but_not_the_mapping():
    inner = _RecordingStream()
    proxy = PooledBufferIO(inner)
    proxy.close(truncate=True)
    assert inner.named("resize") == [("resize", METADATA_SIZE + 500)] and proxy.closed and not inner.named("close")
    inner = _RecordingStream()
    proxy = PooledBufferIO(inner)
    proxy.close(truncate=False)
    assert not inner.named("resize") and proxy.closed


# ---- manager: acquire (test_checkpoint_object_manager.py:102-282, :816-903) -------------------------------------------
def test_acquire_adds_the_metadata_block_to_the_requested_size(manager, tmp_path):
    oid = CheckpointObjectId(str(tmp_path / "metadata_size_test.bin"))
    with manager.acquire_buffer(oid, buffer_size=1024) as buf:
        assert os.path.getsize(str(oid)) == 1024 + METADATA_SIZE
        assert buf.buffer_obj.get_capacity() == 1024 + METADATA_SIZE


def test_acquire_argument_and_collision_errors(manager, tmp_path):
    oid = CheckpointObjectId(str(tmp_path / "o.bin"))
    for size in (0, -100):
        with pytest.raises(ValueError, match="Buffer size must be a positive integer"):
            manager.acquire_buffer(oid, buffer_size=size)
    with pytest.raises(FileExistsError, match=f"File {tmp_path} already exists"):
        manager.acquire_buffer(CheckpointObjectId(str(tmp_path)), buffer_size=1024, overwrite=False)  # a directory
    with manager.acquire_buffer(oid, 100) as buf:
        buf.write(b"data")
    with pytest.raises(FileExistsError, match=f"File {oid} already exists and overwrite=False"):
        manager.acquire_buffer(oid, 100, overwrite=False)
    (tmp_path / "untracked.bin").write_bytes(b"old content nobody registered")
    with manager.acquire_buffer(CheckpointObjectId(str(tmp_path / "untracked.bin")), 64, overwrite=True) as buf:
        buf.write(b"new")
    with manager.get_buffer(CheckpointObjectId(str(tmp_path / "untracked.bin"))) as r:
        assert r.read() == b"new"


def test_acquire_wraps_native_failures(manager, tmp_path, monkeypatch):
    oid = CheckpointObjectId(str(tmp_path / "fail.bin"))

    def broken(*args, **kwargs):
        raise RuntimeError("C++ layer failed")

    monkeypatch.setattr(com_module, "BufferObject", broken)
    with pytest.raises(RuntimeError, match=f"Failed to create buffer for '{oid}'"):
        manager.acquire_buffer(oid, 1024)
    monkeypatch.undo()

    def broken_io(*args, **kwargs):
        raise ValueError("Invalid buffer")

    monkeypatch.setattr(com_module, "BufferIO", broken_io)
    with pytest.raises(RuntimeError, match=f"Failed to create buffer for '{oid}'"):
        manager.acquire_buffer(oid, 1024)


# ---- manager: get / close / delete (:284-771) ----------------------------------------------------------------------------
def test_get_buffer_read_only_or_none(manager, tmp_path):
    oid = CheckpointObjectId(str(tmp_path / "o.bin"))
    with manager.acquire_buffer(oid, 128) as w:
        w.write(b"payload")
    r = manager.get_buffer(oid)
    assert r.is_readonly and r.read() == b"payload"
    manager.close_buffer(r)
    assert r.closed
    manager.close_buffer(r)                                     # again: ignored
    assert manager.get_buffer(CheckpointObjectId(str(tmp_path / "non_existent.bin"))) is None
    assert manager.get_buffer(CheckpointObjectId(str(tmp_path))) is None            # a directory
    (tmp_path / "malformed.bin").write_bytes(b"bad_data")                             # shorter than the metadata block
    assert manager.get_buffer(CheckpointObjectId(str(tmp_path / "malformed.bin"))) is None
    for exc in (ValueError("bad"), RuntimeError("bad"), OSError("bad")):
        with pytest.MonkeyPatch.context() as mp:
            mp.setattr(com_module, "BufferObject", lambda *a, _e=exc, **k: (_ for _ in ()).throw(_e))
            assert manager.get_buffer(oid) is None


def test_close_buffer_and_links(manager, tmp_path):
    target, link, plain = tmp_path / "target.bin", tmp_path / "link.bin", tmp_path / "regular.bin"
    target.write_bytes(bytes(METADATA_SIZE + 10))
    plain.write_bytes(bytes(METADATA_SIZE + 10))
    os.symlink(target, link)
    via_link = manager.get_buffer(CheckpointObjectId(str(link)))
    manager.close_buffer(via_link, skip_close_if_symlink=True)
    assert not via_link.closed                                  # opened through a link: left open
    manager.close_buffer(via_link, skip_close_if_symlink=False)
    assert via_link.closed
    regular = manager.get_buffer(CheckpointObjectId(str(plain)))
    manager.close_buffer(regular, skip_close_if_symlink=True)
    assert regular.closed                                       # a regular file closes either way


def test_close_buffer_truncates_to_what_was_written(manager, tmp_path):
    oid = CheckpointObjectId(str(tmp_path / "trunc.bin"))
    buf = manager.acquire_buffer(oid, 4096)
    buf.write(b"x" * 100)
    assert os.path.getsize(str(oid)) == METADATA_SIZE + 4096
    manager.close_buffer(buf)
    assert os.path.getsize(str(oid)) == METADATA_SIZE + 100

    class Failing(BufferIO):
        def close(self, truncate=True):
            raise OSError("Disk full")

    buf = manager.acquire_buffer(CheckpointObjectId(str(tmp_path / "f.bin")), 64)
    buf.__class__ = Failing
    with pytest.raises(OSError, match="Disk full"):             # a failing close is the caller's to see
        manager.close_buffer(buf)
    BufferIO.close(buf)


def test_delete_object_and_container(manager, tmp_path):
    box = tmp_path / "step-3_ckpt"
    oid = CheckpointObjectId(str(box / "a.distcp"))
    with manager.acquire_buffer(oid, 16) as w:
        w.write(b"a")
    manager.delete_object(oid)
    assert not os.path.exists(str(oid))
    manager.delete_object(oid)                                  # missing: a warning, no error
    broken = CheckpointObjectId(str(tmp_path / "broken_link"))
    os.symlink(tmp_path / "non_existent_target", str(broken))
    assert os.path.lexists(str(broken)) and not os.path.exists(str(broken))
    manager.delete_object(broken)
    assert not os.path.lexists(str(broken))                     # a dangling link is removed too
    with manager.acquire_buffer(CheckpointObjectId(str(box / "b.distcp")), 16) as w:
        w.write(b"b")
    manager.delete_container(CheckpointContainerId(str(box)))
    assert not box.exists()
    manager.delete_container(CheckpointContainerId(str(box)))   # gone already: nothing to do
    empty = tmp_path / "step-4_ckpt"
    empty.mkdir()
    manager.delete_container(CheckpointContainerId(str(empty)))
    assert not empty.exists()
    a_file = tmp_path / "step-5_ckpt"
    a_file.write_text("I am a file, not a container.")
    manager.delete_container(CheckpointContainerId(str(a_file)))
    assert a_file.exists()                                      # a file is not a container: left alone


def test_delete_container_passes_over_files_that_vanish(manager, tmp_path, monkeypatch):
    seen = {}

    def fake_rmtree(path, onerror=None, **kwargs):
        seen["onerror"] = onerror

    box = tmp_path / "step-6_ckpt"
    box.mkdir()
    monkeypatch.setattr(com_module.shutil, "rmtree", fake_rmtree)
    manager.delete_container(CheckpointContainerId(str(box)))
    handler = seen["onerror"]
    exc = FileNotFoundError("file missing")
    handler(None, None, (type(exc), exc, None))                 # swallowed: somebody else deleted it first
    with pytest.raises(ValueError):
        exc = ValueError("some other error")
        handler(None, None, (type(exc), exc, None))

    def denied(path, onerror=None, **kwargs):
        raise OSError("Permission denied")

    monkeypatch.setattr(com_module.shutil, "rmtree", denied)
    with pytest.raises(OSError, match="Permission denied"):
        manager.delete_container(CheckpointContainerId(str(box)))


# ---- manager: the process-wide pool (:906-1035) -----------------------------------------------------------------------
def test_pool_is_created_lazily_once_per_process(manager, tmp_path, monkeypatch):
    created = []

    class CountingPool(BufferPool):
        def __init__(self, **kwargs):
            created.append(kwargs)
            super().__init__(**kwargs)

    monkeypatch.setattr(com_module, "BufferPool", CountingPool)
    cfg = BufferPoolConfig(pool_dir_path=str(tmp_path / "lazy"), rank=0, num_buffers=2, buffer_size=METADATA_SIZE + 64)
    m1, m2 = CheckpointObjectManager(pool_config=cfg), CheckpointObjectManager(pool_config=cfg)
    assert m1._pool_config == cfg and CheckpointObjectManager._worker_pool is None and not created
    assert CheckpointObjectManager(pool_config=None)._get_or_create_buffer_pool() is None
    m1.acquire_buffer(CheckpointObjectId(str(tmp_path / "ck" / "1")), 100).close()
    assert created == [dict(pool_dir_path=str(tmp_path / "lazy"), num_buffers=2, rank=0, buffer_size=METADATA_SIZE + 64)]
    first = CheckpointObjectManager._worker_pool
    m1.acquire_buffer(CheckpointObjectId(str(tmp_path / "ck" / "1")), 100).close()
    m2.acquire_buffer(CheckpointObjectId(str(tmp_path / "ck" / "2")), 100).close()
    assert len(created) == 1 and CheckpointObjectManager._worker_pool is first
    m2.teardown_pool()
    assert CheckpointObjectManager._worker_pool is None and not first.free_buffers and not first.active_buffers


def test_pool_creation_failure_and_pickling(manager, tmp_path, monkeypatch):
    def failing(**kwargs):
        raise Exception("Init failed")

    monkeypatch.setattr(com_module, "BufferPool", failing)
    cfg = BufferPoolConfig(pool_dir_path=str(tmp_path / "fail_init"), rank=0, num_buffers=1, buffer_size=0)
    m = CheckpointObjectManager(pool_config=cfg)
    logged = []

    class Log:
        def exception(self, msg, *args):
            logged.append(msg)

        def __getattr__(self, name):
            return lambda *a, **k: None

    monkeypatch.setattr(com_module, "_LOGGER", Log())
    assert m._get_or_create_buffer_pool() is None
    assert CheckpointObjectManager._worker_pool is None
    assert len(logged) == 1 and "Failed to initialize BufferPool" in logged[0]
    oid = CheckpointObjectId(str(tmp_path / "ck" / "standalone"))
    with m.acquire_buffer(oid, 32) as buf:                      # falls back to a file of its own
        assert isinstance(buf, BufferIO) and not os.path.islink(str(oid))
    CheckpointObjectManager._worker_pool = "fake_pool"
    clone = pickle.loads(pickle.dumps(m))
    assert clone._pool_config == cfg and CheckpointObjectManager._worker_pool == "fake_pool"  # class state untouched
    CheckpointObjectManager._worker_pool = None
