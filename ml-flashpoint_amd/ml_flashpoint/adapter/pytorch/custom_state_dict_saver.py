"""A DCP save cut into three calls - ``generate_plan``, ``write_data``, ``finish_write`` - so that an async framework
can run the middle one in a worker while the training process goes on.  Names, arguments and results are those of the
reference's module (src/ml_flashpoint/adapter/pytorch/custom_state_dict_saver.py:42-227), which the Megatron/NeMo
strategies call.

With the gfx950 saver the blocking work of a save ends inside ``generate_plan``: its last step,
``storage_writer.prepare_write_data_buckets``, lays the object out and enqueues the pack of its image on the
training stream.
"""

from __future__ import annotations

import logging
from typing import NamedTuple

import torch
import torch.distributed as torchdist
from torch.distributed.checkpoint.metadata import STATE_DICT_TYPE, Metadata
from torch.distributed.checkpoint.planner import SavePlan, SavePlanner
from torch.distributed.checkpoint.storage import WriteResult
from torch.distributed.checkpoint.utils import _DistWrapper

from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.core import utils
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
from ml_flashpoint.core.checkpoint_saver import ObjectWriteBucket
from ml_flashpoint.core.mlf_logging import get_logger

_LOGGER = get_logger(__name__)


class _CachedStructure(NamedTuple):
    """What a caller keeps from one save for the next (``cached_ckpt_structure``)."""

    central_plan: SavePlan | None = None  # this rank's share of the global plan
    local_plan: SavePlan | None = None    # this rank's own plan, before the global step
    validated: bool = False               # two consecutive saves produced the same central plan


@utils.log_execution_time(logger=_LOGGER, name="generate_plan", level=logging.INFO)
def generate_plan(
    checkpoint_id: CheckpointContainerId,
    state_dict: STATE_DICT_TYPE,
    storage_writer: MemoryStorageWriter,
    planner: SavePlanner,
    world_dist_wrapper: _DistWrapper,
    cached_ckpt_structure: tuple[SavePlan, SavePlan, bool] | None = None,
) -> tuple[list[ObjectWriteBucket], Metadata | None, SavePlan, SavePlan, bool]:
    """Planning phase: ``(write_buckets, global_metadata, central_plan, local_plan, validated_cache_reuse)``.

    The last three are the next save's ``cached_ckpt_structure``.  As long as the cache is not validated every save
    plans from scratch (local plan, reduce-scatter through the coordinator's global plan, metadata broadcast) and
    compares its central plan with the cached one; once they were equal, later saves skip all three steps and
    ``global_metadata`` comes back as None - the caller already holds the metadata that goes with the cached plan.
    """
    with utils.gc_paused():  # planning allocates ~10 small objects per tensor, none of them cyclic
        cache = _CachedStructure(*cached_ckpt_structure) if cached_ckpt_structure else _CachedStructure()
        coordinator = world_dist_wrapper.is_coordinator
        planner.set_up_planner(state_dict=state_dict, storage_meta=storage_writer.storage_meta(), is_coordinator=coordinator)
        storage_writer.set_up_storage_writer(coordinator)
        if cache.validated and cache.central_plan:
            local_plan = storage_writer.prepare_local_plan(cache.local_plan or planner.create_local_plan())
            central_plan, global_metadata = cache.central_plan, None
        else:
            local_plan = storage_writer.prepare_local_plan(planner.create_local_plan())
            central_plan, global_metadata = _agree_on_plan(local_plan, storage_writer, planner, world_dist_wrapper)
        buckets = storage_writer.prepare_write_data_buckets(checkpoint_id, planner.finish_plan(central_plan), planner)
        expect = getattr(storage_writer, "expect_metadata", None)
        if expect is not None and torchdist.get_node_local_rank(fallback_rank=0) == 0:
            # This process is going to write the metadata object in finish_write, and which object that is, is known
            # now (a validated cache: the one the last planning save produced, which the caller was handed then and
            # hands back to finish_write): the writer may pickle it while the data is on its way.  With several
            # ranks the others' write results are predicted to be those of the previous save.
            saver = getattr(storage_writer, "checkpoint_saver", None)
            if global_metadata is not None:
                _remember(saver, "last_global_metadata", global_metadata)
            expect(global_metadata if global_metadata is not None else getattr(saver, "last_global_metadata", None),
                   others_as_before=bool(world_dist_wrapper.use_dist))
        return buckets, global_metadata, central_plan, local_plan, cache.central_plan == central_plan


def _remember(holder, name: str, value) -> None:
    try:
        setattr(holder, name, value)
    except AttributeError:
        pass


def _agree_on_plan(local_plan, storage_writer, planner, dist: _DistWrapper):
    """Every rank's plan goes to the coordinator, which merges them, lets the writer number them and hands each rank
    its share back; the metadata that the merge produced exists on the coordinator only and is broadcast."""
    merged_metadata = None

    def merge(all_local_plans: list[SavePlan]) -> list[SavePlan]:
        nonlocal merged_metadata
        all_local_plans, merged_metadata = planner.create_global_plan(all_local_plans)
        return storage_writer.prepare_global_plan(all_local_plans)

    with utils.log_execution_time(logger=_LOGGER, name="generate_plan__reduce_scatter_plan"):
        central_plan = dist.reduce_scatter("plan", lambda: local_plan, merge)
    with utils.log_execution_time(logger=_LOGGER, name="generate_plan__broadcast_metadata"):
        return central_plan, dist.broadcast_object(merged_metadata)


@utils.log_execution_time(logger=_LOGGER, name="write_data", level=logging.INFO)
def write_data(
    checkpoint_id: CheckpointContainerId,
    storage_writer: MemoryStorageWriter,
    staged_write_buckets: list[ObjectWriteBucket],
    replicate_after_write: bool,
) -> list[WriteResult]:
    """Write phase, synchronous: the call an async framework runs in its worker."""
    pending = storage_writer.write_staged_data_buckets(checkpoint_id, staged_write_buckets, replicate_after_write)
    return pending.wait()


@utils.log_execution_time(logger=_LOGGER, name="finish_write", level=logging.INFO)
def finish_write(
    checkpoint_id: CheckpointContainerId,
    storage_writer: MemoryStorageWriter,
    global_metadata: Metadata,
    world_dist_wrapper: _DistWrapper,
) -> None:
    """Completion phase, to be called once the write of ``checkpoint_id`` is known to be done on this rank: the
    ranks' write results are gathered on the coordinator and broadcast back, and the first rank of every node
    writes the checkpoint's metadata object."""
    own = storage_writer.get_write_results(checkpoint_id)
    everyones = world_dist_wrapper.gather_object(own)
    with utils.log_execution_time(logger=_LOGGER, name="finish_write__broadcast_results"):
        everyones = world_dist_wrapper.broadcast_object(everyones)
    if torchdist.get_node_local_rank(fallback_rank=0) != 0:
        return
    storage_writer.finish_checkpoint(checkpoint_id=checkpoint_id, metadata=global_metadata, results=everyones)


def _get_local_rank_0_global_ranks() -> list[int]:
    """Global ranks that are rank 0 of their node, assuming every node runs one rank per visible GPU
    (reference: custom_state_dict_saver.py:218-227; nothing calls it there either)."""
    per_node = torch.cuda.device_count()
    return [node * per_node for node in range(utils.get_num_of_nodes())]
