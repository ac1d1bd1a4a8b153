"""``generate_plan`` / ``write_data`` / ``finish_write``, case by case as the reference's suite states them
(tests/adapter/pytorch/test_custom_state_dict_saver.py:57-480), with ``unittest.mock`` writer and planner and a real
single-process ``_DistWrapper``."""

from unittest import mock

import pytest
import torch
from torch.distributed.checkpoint.metadata import (
    BytesStorageMetadata,
    ChunkStorageMetadata,
    Metadata,
    MetadataIndex,
    TensorProperties,
    TensorStorageMetadata,
)
from torch.distributed.checkpoint.planner import SavePlan, SavePlanner, WriteItem, WriteItemType
from torch.distributed.checkpoint.storage import WriteResult
from torch.distributed.checkpoint.utils import _DistWrapper
from torch.futures import Future as TorchFuture

from ml_flashpoint.adapter.pytorch import custom_state_dict_saver
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_saver import ObjectWriteBucket

CID = CheckpointContainerId("/test_checkpoint")


@pytest.fixture
def writer():
    w = mock.MagicMock(spec=MemoryStorageWriter)
    w.get_write_results.return_value = [mock.MagicMock()]
    return w


@pytest.fixture
def planner():
    return mock.MagicMock(spec=SavePlanner)


@pytest.fixture
def dist():
    return _DistWrapper(group=None, use_dist=False, coordinator_rank=0)


def _buckets(tag, base=0):
    return [ObjectWriteBucket(object_id=CheckpointObjectId(f"/test_checkpoint/{tag}_{i}"), object_name=f"{tag}_{i}",
                              bytesio_data=[], tensor_data=[(mock.MagicMock(), torch.tensor([i + base]))])
            for i in range(2)]


def _wire(writer, planner, local_plan, global_plans, metadata):
    planner.create_local_plan.return_value = local_plan
    writer.prepare_local_plan.return_value = local_plan
    planner.create_global_plan.return_value = (global_plans, metadata)
    writer.prepare_global_plan.return_value = global_plans
    planner.finish_plan.return_value = local_plan


# ---- generate_plan (:57-336) ----------------------------------------------------------------------------------------------
def test_generate_plan_call_sequence(writer, planner, dist):
    local_plan = SavePlan([])
    chunk = [ChunkStorageMetadata(offsets=torch.Size([0, 0]), sizes=torch.Size([5, 10]))]
    metadata = Metadata(state_dict_metadata={
        "tensor1": TensorStorageMetadata(size=torch.Size([10, 20]), properties=TensorProperties(dtype=torch.float32), chunks=chunk),
        "tensor2": TensorStorageMetadata(size=torch.Size([30, 40]), properties=TensorProperties(dtype=torch.float32), chunks=chunk),
        "dir1/shard_0_0": BytesStorageMetadata(),
    })
    _wire(writer, planner, local_plan, [local_plan], metadata)
    writer.prepare_write_data_buckets.return_value = expected = _buckets("obj")
    order = mock.MagicMock()
    for name, target in (("set_up_planner", planner.set_up_planner), ("set_up_storage_writer", writer.set_up_storage_writer),
                         ("create_local_plan", planner.create_local_plan), ("prepare_local_plan", writer.prepare_local_plan),
                         ("create_global_plan", planner.create_global_plan), ("prepare_global_plan", writer.prepare_global_plan),
                         ("finish_plan", planner.finish_plan), ("prepare_write_data_buckets", writer.prepare_write_data_buckets)):
        order.attach_mock(target, name)
    buckets, got_metadata, _, _, reused = custom_state_dict_saver.generate_plan(CID, {"model": "test"}, writer, planner, dist)
    assert [c[0] for c in order.mock_calls] == ["set_up_planner", "set_up_storage_writer", "create_local_plan",
                                                "prepare_local_plan", "create_global_plan", "prepare_global_plan",
                                                "finish_plan", "prepare_write_data_buckets"]
    writer.prepare_local_plan.assert_called_once_with(local_plan)
    planner.create_global_plan.assert_called_once_with([local_plan])
    writer.prepare_global_plan.assert_called_once_with([local_plan])
    planner.finish_plan.assert_called_once_with(local_plan)
    writer.prepare_write_data_buckets.assert_called_once_with(CID, local_plan, planner)
    assert buckets == expected and got_metadata == metadata and reused is False


def test_generate_plan_with_a_validated_cache_skips_planning(writer, planner, dist):
    cached_plan = SavePlan([WriteItem(index=MetadataIndex("cached"), type=WriteItemType.TENSOR)])
    planner.finish_plan.return_value = cached_plan
    writer.prepare_write_data_buckets.return_value = []
    with mock.patch.object(dist, "reduce_scatter") as reduce_scatter, mock.patch.object(dist, "broadcast_object") as broadcast:
        _, metadata, central, _, reused = custom_state_dict_saver.generate_plan(
            CID, {"model": "test"}, writer, planner, dist, cached_ckpt_structure=(cached_plan, SavePlan([]), True))
        reduce_scatter.assert_not_called()
        broadcast.assert_not_called()
    assert metadata is None and reused is True and central is cached_plan
    planner.create_local_plan.assert_not_called()
    planner.finish_plan.assert_called_once_with(cached_plan)


def test_generate_plan_validates_an_unvalidated_cache(writer, planner, dist):
    local_plan = SavePlan([])
    _wire(writer, planner, local_plan, [local_plan], None)
    writer.prepare_write_data_buckets.return_value = []
    with mock.patch.object(dist, "reduce_scatter", return_value=local_plan), \
            mock.patch.object(dist, "broadcast_object", return_value=None):
        *_, reused = custom_state_dict_saver.generate_plan(CheckpointContainerId("/test"), {}, writer, planner, dist,
                                                           cached_ckpt_structure=(local_plan, None, False))
    assert reused is True                                      # same central plan twice in a row
    different = SavePlan([WriteItem(index=MetadataIndex("other"), type=WriteItemType.TENSOR)])
    *_, reused = custom_state_dict_saver.generate_plan(CheckpointContainerId("/test"), {}, writer, planner, dist,
                                                       cached_ckpt_structure=(different, None, False))
    assert reused is False


def test_generate_plan_collectives(writer, planner, dist):
    local_plan = SavePlan([WriteItem(index=MetadataIndex("local_item"), type=WriteItemType.TENSOR)])
    metadata = Metadata(state_dict_metadata={"test_key": "test_value"})
    _wire(writer, planner, local_plan, [local_plan], metadata)
    scattered = SavePlan([WriteItem(index=MetadataIndex("scattered_item"), type=WriteItemType.BYTE_IO)])
    planner.finish_plan.return_value = scattered
    broadcast_result = Metadata(state_dict_metadata={"test_other_key": "test_other_value", "a": 2})

    def run_reduce_scatter(step, map_fun, reduce_fun):          # what the single-process wrapper does
        return reduce_fun([map_fun()])[0] and scattered

    with mock.patch.object(dist, "reduce_scatter", side_effect=run_reduce_scatter) as reduce_scatter, \
            mock.patch.object(dist, "broadcast_object", return_value=broadcast_result) as broadcast:
        _, got_metadata, central, _, _ = custom_state_dict_saver.generate_plan(CID, {"model": "test"}, writer, planner, dist)
        reduce_scatter.assert_called_once()
        assert reduce_scatter.call_args[0][0] == "plan"
        broadcast.assert_called_once_with(metadata)            # the coordinator's metadata goes out to every rank
    assert got_metadata == broadcast_result and central is scattered
    planner.finish_plan.assert_called_once_with(scattered)


def test_generate_plan_result_shape(writer, planner, dist):
    _wire(writer, planner, SavePlan([]), [SavePlan([])], None)
    writer.prepare_write_data_buckets.return_value = []
    result = custom_state_dict_saver.generate_plan(CID, {"model": "test"}, writer, planner, dist)
    assert isinstance(result, tuple) and len(result) == 5
    assert result[0] == [] and result[1] is None and result[2] == SavePlan([]) and result[3] == SavePlan([])
    assert result[4] is False
    writer.prepare_write_data_buckets.return_value = expected = _buckets("obj_ret", base=10)
    assert custom_state_dict_saver.generate_plan(CID, {"model": "test"}, writer, planner, dist)[0] == expected


# ---- write_data (:338-382) -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("replicate", [True, False])
def test_write_data_waits_for_the_writer(writer, replicate):
    staged = [mock.MagicMock()]
    done = TorchFuture()
    expected = [WriteResult(index=MetadataIndex("a"), size_in_bytes=10, storage_data="data_a"),
                WriteResult(index=MetadataIndex("b"), size_in_bytes=20, storage_data="data_b")]
    done.set_result(expected)
    writer.write_staged_data_buckets.return_value = done
    assert custom_state_dict_saver.write_data(CID, writer, staged, replicate_after_write=replicate) == expected
    writer.write_staged_data_buckets.assert_called_once_with(CID, staged, replicate)


# ---- finish_write (:384-455) -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("results", [[mock.sentinel.result], None, []], ids=["some", "none", "empty"])
def test_finish_write_on_node_local_rank_0(writer, dist, results):
    metadata = Metadata(state_dict_metadata={})
    writer.get_write_results.return_value = results
    with mock.patch("torch.distributed.get_node_local_rank", return_value=0):
        custom_state_dict_saver.finish_write(CID, writer, metadata, dist)
    writer.get_write_results.assert_called_once_with(CID)
    writer.finish_checkpoint.assert_called_once_with(checkpoint_id=CID, metadata=metadata, results=[results])
    writer.finish.assert_not_called()


def test_finish_write_elsewhere_writes_nothing(writer, dist):
    with mock.patch("torch.distributed.get_node_local_rank", return_value=1):
        custom_state_dict_saver.finish_write(CID, writer, Metadata(state_dict_metadata={}), dist)
    writer.finish_checkpoint.assert_not_called()
    writer.finish.assert_not_called()


# ---- node-leader ranks (:457-480) --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("num_gpus, num_nodes, expected",
                         [(8, 1, [0]), (8, 2, [0, 8]), (4, 4, [0, 4, 8, 12]), (1, 8, [0, 1, 2, 3, 4, 5, 6, 7])])
def test_node_leader_ranks(num_gpus, num_nodes, expected):
    with mock.patch("torch.cuda.device_count", return_value=num_gpus), \
            mock.patch("ml_flashpoint.core.utils.get_num_of_nodes", return_value=num_nodes):
        assert custom_state_dict_saver._get_local_rank_0_global_ranks() == expected
