"""Checkpoint identifier types, case by case as the reference's suite states them
(tests/core/test_checkpoint_id_types.py:22-329), and two cases of its native-object binding suite that nothing
else here covers (tests/checkpoint_object_manager/buffer_object/test_buffer_object_bindings.py:110-130, :181-198)."""

import pytest

from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId

BOTH = pytest.mark.parametrize("cls", [CheckpointObjectId, CheckpointContainerId])


@BOTH
def test_creation_and_normalisation(cls):
    assert str(cls("/valid/path/to/object")) == "/valid/path/to/object"
    assert str(cls("/valid/path/to/object/")) == "/valid/path/to/object"      # trailing slash dropped
    assert cls("/test/string").data == "/test/string"
    for bad in ("invalid/path", "/", "//", "///", "////", "/////", "/a//b"):
        with pytest.raises(ValueError):
            cls(bad)
    for bad in ("/a/b./c", "/a/b."):
        with pytest.raises(ValueError, match="Path segment cannot end with a '.'"):
            cls(bad)


def test_container_specific_messages():
    for root in ("/", "//", "///"):
        with pytest.raises(ValueError, match="CheckpointContainerId cannot be the root path '/'"):
            CheckpointContainerId(root)
    with pytest.raises(ValueError, match="Path segment cannot be empty"):
        CheckpointContainerId("/a//b")


@BOTH
def test_equality_with_ids_and_strings(cls):
    assert cls("/same/path") == cls("/same/path") and cls("/same/path") != cls("/different/path")
    assert cls("/same/path") == "/same/path" and cls("/same/path") != "/different/path"


def test_parents():
    obj = CheckpointObjectId("/a/b/c/d")
    for levels, want in ((1, "/a/b/c"), (2, "/a/b"), (3, "/a")):
        parent = obj.get_parent(levels_up=levels)
        assert isinstance(parent, CheckpointContainerId) and str(parent) == want
    assert str(obj.get_parent()) == "/a/b/c"
    assert CheckpointObjectId("/a/b").get_parent(levels_up=2) is None         # would be the root
    assert CheckpointObjectId("/a/b/c").get_parent(levels_up=3) is None
    assert CheckpointObjectId("/a").get_parent(levels_up=1) is None
    for bad in (0, -1):
        with pytest.raises(ValueError):
            CheckpointObjectId("/a/b/c").get_parent(levels_up=bad)
    box = CheckpointContainerId("/a/b/c")
    assert isinstance(box.get_parent(), CheckpointContainerId) and str(box.get_parent()) == "/a/b"
    assert CheckpointContainerId("/a").get_parent() is None
    assert CheckpointContainerId("/a/b").get_parent(levels_up=2) is None


def test_object_id_from_container():
    parent = CheckpointContainerId("/base/path")
    made = CheckpointObjectId.from_container(parent, "object_name")
    assert isinstance(made, CheckpointObjectId) and str(made) == "/base/path/object_name"
    assert str(CheckpointObjectId.from_container(CheckpointContainerId("/base/path/"), "/object_name/")) == (
        "/base/path/object_name"
    )
    assert str(CheckpointObjectId.from_container(parent, "obj-name.ext=1")) == "/base/path/obj-name.ext=1"
    assert str(CheckpointObjectId.from_container(parent, "  object_name  ")) == "/base/path/object_name"
    with pytest.raises(TypeError):
        CheckpointObjectId.from_container("/base/path", "object_name")
    for bad in ("", "/", "//", "  ", ".", "..", "..."):
        with pytest.raises(ValueError):
            CheckpointObjectId.from_container(parent, bad)


def test_container_children():
    parent = CheckpointContainerId("/base/path")
    assert str(CheckpointContainerId.create_child(parent, "child")) == "/base/path/child"
    assert str(CheckpointContainerId.create_child(CheckpointContainerId("/base/path/"), "/child/")) == "/base/path/child"
    assert str(CheckpointContainerId.create_child(parent, "")) == "/base/path"   # no name: the parent itself
    assert str(CheckpointContainerId.create_child(parent, "/")) == "/base/path"
    with pytest.raises(TypeError):
        CheckpointContainerId.create_child("/base/path", "child")


def test_version_container_names():
    pattern = CheckpointContainerId.get_version_container_pattern()
    assert pattern.match("step-123_ckpt")
    assert not pattern.match("step-123_checkpoint") and not pattern.match("mystep-123_ckpt")
    dirty = CheckpointContainerId.get_dirty_version_checkpoint_container_pattern()
    for name in ("step-123_ckpt_unfinished", "step-123_ckpt_rank0__unfinished", "step-123_ckpt_rank0_unfinished"):
        assert dirty.match(name)
    for name in ("step-123_ckpt", "step-123_checkpoint", "mystep-123_ckpt"):
        assert not dirty.match(name)
    assert CheckpointContainerId.format_version_container(123) == "step-123_ckpt"
    assert CheckpointContainerId.format_version_container(-1) == "step--1_ckpt"
    assert CheckpointContainerId.format_version_container(123.0) == "step-123.0_ckpt"
    assert CheckpointContainerId.parse_version_container_step("step-123_ckpt") == 123
    for name in ("invalid-step", "step-123_ckpt_extra", "step--1_ckpt"):
        assert CheckpointContainerId.parse_version_container_step(name) is None
    for bad in (123, None):
        with pytest.raises(TypeError):
            CheckpointContainerId.parse_version_container_step(bad)


# ---- native object ------------------------------------------------------------------------------------------------------
def test_any_file_opens_read_only_and_reopening_is_safe(tmp_path):
    path = tmp_path / "reopen_test.bin"
    path.write_bytes(b"initial data")                      # not a checkpoint object: the native layer does not care
    bo = BufferObject(str(path))
    bo = BufferObject(str(path))
    bo = BufferObject(str(path))                           # earlier instances are released as they are replaced
    assert not bo.closed and bo.is_readonly
    mv = memoryview(bo)
    assert mv.readonly and mv == b"initial data"
    with pytest.raises(TypeError):
        mv[0] = 65
    mv.release()
    bo.close()
    assert bo.closed
