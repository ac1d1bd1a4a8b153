"""BufferIO behaviour, case by case as the reference's own suite states it
(tests/checkpoint_object_manager/test_buffer_io.py:137-1170, read as text and restated against the real native
buffer object; the reference also runs most of them against a Python mock, which has no counterpart here).
Messages and exception types are part of the interface: adapters and user code match on them."""

import io

import pytest

from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE, BufferMetadataType
from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject

CLOSED = "I/O operation on a closed BufferIO object"
READ_ONLY = "Operation 'write' is not supported in read-only mode"


@pytest.fixture
def rw_obj(tmp_path):
    obj = BufferObject(str(tmp_path / "writable_test.bin"), METADATA_SIZE + 1024, overwrite=True)
    yield obj
    if not obj.closed:
        obj.close()


@pytest.fixture
def ro_obj(tmp_path):
    path = str(tmp_path / "readonly_test.bin")
    with BufferIO(BufferObject(path, METADATA_SIZE + 512, overwrite=True)) as w:
        w.write(b"some pre-existing data")
    obj = BufferObject(path)
    yield obj
    if not obj.closed:
        obj.close()


# ---- initialisation (:137-163) -----------------------------------------------------------------------------------
def test_initialisation_states(rw_obj, ro_obj, tmp_path):
    bio = BufferIO(rw_obj)
    assert bio.buffer_obj is rw_obj and bio.tell() == 0 and bio.closed is False and bio.is_readonly is False
    bio = BufferIO(ro_obj)
    assert bio.buffer_obj is ro_obj and bio.tell() == 0 and bio.closed is False and bio.is_readonly is True
    small = BufferObject(str(tmp_path / "small_test.bin"), METADATA_SIZE - 1, overwrite=True)
    with pytest.raises(ValueError, match=f"Buffer size must be at least {METADATA_SIZE} bytes"):
        BufferIO(small)
    small.close()
    rw_obj.close()
    with pytest.raises(ValueError, match="Cannot initialize BufferIO with a closed BufferObject"):
        BufferIO(rw_obj)


# ---- write (:166-277) ----------------------------------------------------------------------------------------------
def test_write_updates_state_and_lands_after_the_metadata_block(rw_obj):
    bio = BufferIO(rw_obj)
    assert bio.write(b"hello world") == 11 and bio.tell() == 11
    mv = memoryview(rw_obj)
    assert bytes(mv[METADATA_SIZE : METADATA_SIZE + 11]) == b"hello world"
    assert BufferMetadataType.from_buffer(mv).len_written_data == 11
    assert bio.write(b"") == 0 and bio.tell() == 11                 # zero bytes: a no-op
    assert bio.write(b"-a") == 2 and bio.write(b"-bc") == 3 and bio.tell() == 16  # chunks accumulate
    bio.seek(0)
    assert bio.read() == b"hello world-a-bc"


def test_write_errors(rw_obj, ro_obj):
    with pytest.raises(TypeError, match=READ_ONLY):
        BufferIO(ro_obj).write(b"This should fail.")
    bio = BufferIO(rw_obj)
    bio.seek(1000)  # 24 bytes left
    with pytest.raises(ValueError, match="Write operation exceeds buffer capacity"):
        bio.write(b"This data is too long to fit.")
    bio.close()
    with pytest.raises(ValueError, match=CLOSED):
        bio.write(b"x")


def test_write_after_seeking_back_does_not_shrink_the_written_length(rw_obj):
    bio = BufferIO(rw_obj)
    bio.write(b"0123456789")
    bio.seek(2)
    bio.write(b"AB")
    assert bio.tell() == 4 and bio._metadata.len_written_data == 10
    bio.seek(0)
    assert bio.read() == b"01AB456789"


# ---- next_buffer_slice (:279-337) -------------------------------------------------------------------------------------
def test_next_buffer_slice(rw_obj, ro_obj):
    bio = BufferIO(rw_obj)
    bio.write(b"prefix")
    mv = bio.next_buffer_slice(10)
    assert isinstance(mv, memoryview) and len(mv) == 10 and not mv.readonly
    mv[:] = b"0123456789"
    assert bio.tell() == 16
    assert BufferMetadataType.from_buffer(memoryview(rw_obj)).len_written_data == 16
    bio.seek(6)
    assert bio.read(10) == b"0123456789"
    with pytest.raises(ValueError, match="Size must be non-negative"):
        bio.next_buffer_slice(-1)
    bio.seek(0)
    with pytest.raises(ValueError, match="exceeds buffer capacity"):
        bio.next_buffer_slice(len(memoryview(rw_obj)) - METADATA_SIZE + 1)
    with pytest.raises(TypeError, match=READ_ONLY):
        BufferIO(ro_obj).next_buffer_slice(10)
    mv.release()
    bio.close()
    with pytest.raises(ValueError, match=CLOSED):
        bio.next_buffer_slice(10)


# ---- read (:341-430) -----------------------------------------------------------------------------------------------
def test_read_cases(rw_obj, ro_obj):
    bio = BufferIO(rw_obj)
    bio.write(b"0123456789abcdef")
    bio.seek(0)
    assert bio.read(4) == b"0123" and bio.tell() == 4
    assert bio.read(0) == b"" and bio.tell() == 4            # read(0): nothing, position unchanged
    assert bio.read() == b"456789abcdef" and bio.tell() == 16  # no size: all that is left
    assert bio.read(10) == b"" and bio.read() == b""         # at the end
    bio.seek(10)
    assert bio.read(100) == b"abcdef"                        # more than available: what is left
    assert BufferIO(ro_obj).read() == b"some pre-existing data"
    bio.close()
    with pytest.raises(ValueError, match=CLOSED):
        bio.read()


# ---- readinto (:432-527) -------------------------------------------------------------------------------------------
def test_readinto_cases(rw_obj):
    bio = BufferIO(rw_obj)
    bio.write(b"some data")
    bio.seek(0)
    dest = bytearray(4)
    assert bio.readinto(dest) == 4 and bytes(dest) == b"some" and bio.tell() == 4
    big = bytearray(20)
    assert bio.readinto(big) == 5 and bytes(big[:5]) == b" data" and bytes(big[5:]) == bytes(15)
    assert bio.readinto(bytearray(8)) == 0                   # at the end
    bio.seek(4)
    assert bio.readinto(bytearray(0)) == 0 and bio.tell() == 4
    bio.seek(0)
    pattern = r"readinto\(\) argument must be a writable bytes-like object"
    with pytest.raises(TypeError, match=pattern):
        bio.readinto(memoryview(bytearray(10)).toreadonly())
    with pytest.raises(TypeError, match=pattern):
        bio.readinto(b" " * 10)
    bio.close()
    with pytest.raises(ValueError, match=CLOSED):
        bio.readinto(bytearray(10))


# ---- seek / tell (:530-623, :760-772) ---------------------------------------------------------------------------------
def test_seek_and_tell(rw_obj):
    bio = BufferIO(rw_obj)
    content = b"data with a known length of 30"
    bio.write(content)
    assert bio.seek(5) == 5 and bio.tell() == 5
    assert bio.seek(3, io.SEEK_CUR) == 8 and bio.seek(-2, io.SEEK_CUR) == 6
    assert bio.seek(-10, io.SEEK_END) == 20 and bio.tell() == 20   # END = end of the written data
    with pytest.raises(ValueError, match="Negative seek position is not allowed"):
        bio.seek(-1, io.SEEK_SET)
    bio.seek(5)
    with pytest.raises(ValueError, match="Negative seek position is not allowed"):
        bio.seek(-10, io.SEEK_CUR)
    for whence in (3, -1):
        with pytest.raises(ValueError, match="invalid whence value"):
            bio.seek(0, whence)
    bio.seek(2)
    bio.read(2)
    assert bio.tell() == 4
    bio.close()
    with pytest.raises(ValueError, match=CLOSED):
        bio.seek(0)


def test_write_after_seeking_past_the_end_extends_the_written_data(rw_obj):
    bio = BufferIO(rw_obj)
    bio.write(b"0123456789")
    bio.seek(10, io.SEEK_END)
    assert bio.tell() == 20
    bio.write(b"XYZ")
    assert bio.tell() == 23 and bio._metadata.len_written_data == 23
    bio.seek(0)
    assert bio.read() == b"0123456789" + bytes(10) + b"XYZ"


# ---- close / flush / context manager (:626-788) -----------------------------------------------------------------------
def test_close_with_and_without_truncation(tmp_path):
    path = str(tmp_path / "trunc.bin")
    bio = BufferIO(BufferObject(path, METADATA_SIZE + 1024, overwrite=True))
    bio.write(b"twelve bytes")
    bio.close(truncate=True)
    assert bio.closed and (tmp_path / "trunc.bin").stat().st_size == METADATA_SIZE + 12
    bio.close()
    bio.close(truncate=True)                                   # closing again is safe
    path2 = str(tmp_path / "keep.bin")
    bio = BufferIO(BufferObject(path2, METADATA_SIZE + 1024, overwrite=True))
    bio.write(b"twelve bytes")
    bio.close(truncate=False)
    assert (tmp_path / "keep.bin").stat().st_size == METADATA_SIZE + 1024
    ro = BufferIO(BufferObject(path))                          # a read-only stream ignores the truncation request
    ro.close(truncate=True)
    assert (tmp_path / "trunc.bin").stat().st_size == METADATA_SIZE + 12


def test_flush_and_context_manager(rw_obj, tmp_path):
    bio = BufferIO(rw_obj)
    bio.flush()                                                # a no-op on an open stream
    bio.close()
    with pytest.raises(ValueError, match=CLOSED):
        bio.flush()
    with BufferIO(BufferObject(str(tmp_path / "a.bin"), METADATA_SIZE + 64, overwrite=True)) as b1:
        b1.write(b"data")
    assert b1.closed
    with pytest.raises(ValueError, match="Something went wrong"):
        with BufferIO(BufferObject(str(tmp_path / "b.bin"), METADATA_SIZE + 64, overwrite=True)) as b2:
            raise ValueError("Something went wrong")
    assert b2.closed


# ---- signature (:987-1017) -----------------------------------------------------------------------------------------------
def test_format_signature(rw_obj):
    bio = BufferIO(rw_obj)
    assert bio.format_signature == b""                         # nothing is written unless asked for
    assert bytes(memoryview(rw_obj)[8:16]) == bytes(8)
    bio.set_format_signature(b"CUSTOMSG")
    assert bio.format_signature == b"CUSTOMSG"
    assert bytes(memoryview(rw_obj)[8:16]) == b"CUSTOMSG"      # eight bytes right behind the written length
    with pytest.raises(ValueError, match="Format signature must be at most 8 bytes"):
        bio.set_format_signature(b"TOO_LONG_SIGNATURE")


# ---- resize (:1020-1125) -----------------------------------------------------------------------------------------------
def test_resize_cases(tmp_path):
    path = str(tmp_path / "resize.bin")
    initial = METADATA_SIZE + 1024
    with BufferIO(BufferObject(path, initial, overwrite=True)) as bio:
        assert bio.buffer_obj.get_capacity() == initial
        data = b"some data before resize"
        bio.write(data)
        bio.resize(initial * 2)
        assert bio.buffer_obj.get_capacity() == initial * 2 and len(bio._mv) == initial * 2
        bio.seek(0)
        assert bio.read(len(data)) == data                       # content survives
        bio.seek(initial - METADATA_SIZE)                        # the end of the old area
        assert bio.write(b"new data") == 8                       # the new area is writable
        with pytest.raises(ValueError, match=f"New size must be at least {METADATA_SIZE} bytes, got 0"):
            bio.resize(0)
        with pytest.raises(ValueError, match=f"New size must be at least {METADATA_SIZE} bytes"):
            bio.resize(METADATA_SIZE - 1)
        bio.resize(METADATA_SIZE)
        assert bio.buffer_obj.get_capacity() == METADATA_SIZE and len(bio._mv) == METADATA_SIZE
        bio.resize(METADATA_SIZE + 1)
        assert bio.buffer_obj.get_capacity() == METADATA_SIZE + 1 and len(bio._mv) == METADATA_SIZE + 1
    with pytest.raises(ValueError, match=CLOSED):
        bio.resize(METADATA_SIZE + 2048)
    ro = BufferIO(BufferObject(path))
    with pytest.raises(TypeError, match=READ_ONLY):
        ro.resize(METADATA_SIZE + 2048)
    ro.close()


# ---- end to end (:791-984) ---------------------------------------------------------------------------------------------
def test_lifecycle_write_truncate_reopen(tmp_path):
    path = str(tmp_path / "e2e.bin")
    with BufferIO(BufferObject(path, METADATA_SIZE + 4096, overwrite=True)) as w:
        w.write(b"part one, ")
        w.write(b"part two")
        w.seek(0)
        w.write(b"PART")                                        # overwrite inside the written data
    assert (tmp_path / "e2e.bin").stat().st_size == METADATA_SIZE + 18   # the context exit truncates
    with BufferIO(BufferObject(path)) as r:
        assert r.is_readonly and r.read() == b"PART one, part two"
        r.seek(5)
        buf = bytearray(3)
        assert r.readinto(buf) == 3 and bytes(buf) == b"one"
        with pytest.raises(TypeError, match=READ_ONLY):
            r.write(b"x")
    with pytest.raises(RuntimeError):                           # exists, and overwrite was not asked for
        BufferObject(path, METADATA_SIZE + 16, overwrite=False)
    (tmp_path / "empty.bin").touch()
    with pytest.raises(RuntimeError):
        BufferObject(str(tmp_path / "empty.bin"))               # an empty file cannot be mapped
    with pytest.raises(RuntimeError):
        BufferObject(str(tmp_path))                             # nor can a directory
