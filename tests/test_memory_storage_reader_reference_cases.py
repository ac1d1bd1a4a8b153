"""``MemoryStorageReader`` behaviour, case by case as the reference's suite states it
(tests/adapter/pytorch/test_memory_storage_reader.py:50-376): requests are grouped by object file and handed to the
loader, one call per file; the legacy ``torch.save`` record of its end-to-end case is read through the CPU branch
of the real loader (no GPU needed: the target is a host tensor)."""

from pathlib import Path
from unittest import mock

import pytest
import torch
from torch.distributed.checkpoint.filesystem import FileSystem, _StorageInfo
from torch.distributed.checkpoint.metadata import (
    BytesStorageMetadata,
    ChunkStorageMetadata,
    Metadata,
    MetadataIndex,
    StorageMeta,
    TensorProperties,
    TensorStorageMetadata,
)
from torch.distributed.checkpoint.planner import LoadItemType, LoadPlan, LoadPlanner, ReadItem

from ml_flashpoint.adapter.pytorch import memory_storage_reader as reader_module
from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader


def _real_loader():
    return DefaultMLFlashpointCheckpointLoader(
        CheckpointObjectManager(), None, global_rank_getter=lambda: 0, local_rank_getter=lambda: 0,
        broadcast_object_list_func=lambda *a, **k: None, all_gather_object_func=lambda *a, **k: None,
        world_size_getter=lambda: 1)


def _req(index, offsets=(0,), lengths=(1,)):
    return ReadItem(type=LoadItemType.TENSOR, storage_index=MetadataIndex(index), storage_offsets=offsets,
                    lengths=lengths, dest_index=(0,), dest_offsets=(0,))


def test_construction_and_reset(monkeypatch):
    loader = _real_loader()
    reader = MemoryStorageReader("/some/test/path", checkpoint_loader=loader)
    assert reader._path == "/some/test/path" and reader._checkpoint_container_id == CheckpointContainerId("/some/test/path")
    assert reader._checkpoint_loader is loader and reader._storage_data is None
    asked = []
    monkeypatch.setattr(reader_module, "generate_hfid", lambda prefix: asked.append(prefix) or "new_load_id")
    reader.reset("/new/path")
    assert reader._path == "/new/path" and reader._checkpoint_container_id == CheckpointContainerId("/new/path")
    assert asked == ["memreaderload"] and reader._load_id == "new_load_id"
    reader.reset(Path("/new_path"))                           # path-like ids are accepted
    assert reader._path == Path("/new_path") and reader._checkpoint_container_id == CheckpointContainerId("/new_path")


def test_read_data_groups_requests_by_object(tmp_path):
    loader = mock.MagicMock()
    reader = MemoryStorageReader(path=str(tmp_path), checkpoint_loader=loader)
    reader._storage_data = {
        MetadataIndex("0"): _StorageInfo("file1.pt", 0, 10),
        MetadataIndex("1"): _StorageInfo("file2.pt", 0, 20),
        MetadataIndex("2"): _StorageInfo("file1.pt", 10, 30),
    }
    req1, req2, req3 = _req("0"), _req("1"), _req("2")
    planner = mock.MagicMock()
    done = reader.read_data(LoadPlan(items=[req1, req2, req3]), planner)
    assert done.wait() is None and loader.read_data.call_count == 2
    calls = {c.args[0].data: c.args for c in loader.read_data.call_args_list}
    first, second = calls[str(tmp_path / "file1.pt")], calls[str(tmp_path / "file2.pt")]
    assert isinstance(first[0], CheckpointObjectId)
    assert first[1] == [req1, req3] and first[2] is planner and first[3] is reader._storage_data
    assert second[1] == [req2] and second[2] is planner and second[3] is reader._storage_data


def test_read_data_with_nothing_to_read_and_with_a_failing_loader(tmp_path):
    loader = mock.MagicMock()
    reader = MemoryStorageReader(path=str(tmp_path), checkpoint_loader=loader)
    reader._storage_data = {MetadataIndex("0"): _StorageInfo("file1.pt", 0, 10)}
    with mock.patch("torch.distributed.is_initialized", return_value=True), \
            mock.patch("torch.distributed.get_rank", return_value=0):
        reader.read_data(LoadPlan(items=[]), mock.MagicMock())
    loader.read_data.assert_not_called()
    loader.read_data.side_effect = RuntimeError("Loader failed")
    with pytest.raises(RuntimeError, match="Loader failed"):
        reader.read_data(LoadPlan(items=[_req("0")]), mock.MagicMock())
    assert loader.read_data.called


def test_read_data_with_nothing_to_read_outside_a_process_group(tmp_path):
    """No process group (a single-process ``no_dist`` load) must not turn the informational log line of an empty
    plan into an error."""
    reader = MemoryStorageReader(path=str(tmp_path), checkpoint_loader=mock.MagicMock())
    reader._storage_data = {}
    assert not torch.distributed.is_initialized()
    assert reader.read_data(LoadPlan(items=[]), mock.MagicMock()).wait() is None


def test_read_data_end_to_end_with_a_legacy_record(tmp_path):
    manager = CheckpointObjectManager()
    reader = MemoryStorageReader(path=str(tmp_path), checkpoint_loader=_real_loader())
    saved = torch.randn(2, 3)
    with manager.acquire_buffer(CheckpointObjectId(str(tmp_path / "file1.pt")), buffer_size=saved.nbytes * 100) as buffer:
        torch.save(saved, buffer)                              # no signature set: the loader must fall back to torch.load
        length = buffer.tell()
    assert length > 0
    reader._storage_data = {MetadataIndex("0"): _StorageInfo(relative_path="file1.pt", offset=0, length=length)}
    req = _req("0", offsets=(0, 0), lengths=(2, 3))
    planner = mock.MagicMock(spec=LoadPlanner)
    target = torch.empty_like(saved)
    planner.resolve_tensor.side_effect = lambda item: target if item == req else (_ for _ in ()).throw(ValueError(item))
    reader.read_data(LoadPlan(items=[req]), planner)
    planner.resolve_tensor.assert_called_once_with(req)
    assert torch.equal(target, saved)
    planner.commit_tensor.assert_called_once()
    committed = planner.commit_tensor.call_args.args
    assert committed[0] == req and torch.equal(committed[1], target)


def test_validate_checkpoint_id_is_the_file_system_rule():
    with mock.patch.object(FileSystem, "validate_checkpoint_id") as validate:
        MemoryStorageReader.validate_checkpoint_id("/test/path")
        validate.assert_called_once_with("/test/path")


def test_read_metadata_stamps_the_load_id(tmp_path):
    loader = mock.MagicMock()
    reader = MemoryStorageReader(path=str(tmp_path), checkpoint_loader=loader)
    reader._load_id = "test_load_id"
    chunk = [ChunkStorageMetadata(offsets=torch.Size([0, 0]), sizes=torch.Size([5, 10]))]
    expected = Metadata(
        state_dict_metadata={
            "tensor1": TensorStorageMetadata(size=torch.Size([10, 20]), properties=TensorProperties(dtype=torch.float32), chunks=chunk),
            "tensor2": TensorStorageMetadata(size=torch.Size([30, 40]), properties=TensorProperties(dtype=torch.float32), chunks=chunk),
            "dir1/shard_0_0": BytesStorageMetadata(),
        },
        storage_meta=StorageMeta(),
    )
    loader.read_metadata.return_value = expected
    got = reader.read_metadata()
    loader.read_metadata.assert_called_once_with(CheckpointContainerId(str(tmp_path)))
    assert got == expected and got.storage_meta.load_id == "test_load_id"


def test_set_up_storage_reader(tmp_path):
    reader = MemoryStorageReader(path=str(tmp_path), checkpoint_loader=_real_loader())
    storage_data = {MetadataIndex("0"): _StorageInfo(relative_path="file1.pt", offset=0, length=100)}
    reader.set_up_storage_reader(Metadata(state_dict_metadata={}, storage_data=storage_data), is_coordinator=True)
    assert reader._storage_data == storage_data
    with pytest.raises(ValueError, match="metadata.storage_data cannot be None."):
        reader.set_up_storage_reader(Metadata(state_dict_metadata={}, storage_data=None), is_coordinator=True)
    plan = LoadPlan(items=[])
    assert reader.prepare_local_plan(plan) is plan and reader.prepare_global_plan([plan]) == [plan]
