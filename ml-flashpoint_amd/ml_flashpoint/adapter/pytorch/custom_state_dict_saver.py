"""DCP's ``save()`` cut into three calls - plan, write, finish - so that an async framework can run the write in a
worker while the training process goes on (interface and semantics of the reference's
src/ml_flashpoint/adapter/pytorch/custom_state_dict_saver.py:42-215, itself derived from torch's state_dict_saver).

With the gfx950 saver the blocking work of a save ends inside ``generate_plan``: its last step,
``prepare_write_data_buckets``, enqueues the pack of the checkpoint image on the training stream.
"""

import logging

import torch
from torch import distributed as torchdist
from torch.distributed.checkpoint import state_dict_saver as torchdistsaver
from torch.distributed.checkpoint.planner import SavePlan
from torch.distributed.checkpoint.storage import WriteResult
from torch.distributed.checkpoint.utils import _DistWrapper

from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.core import utils
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
from ml_flashpoint.core.checkpoint_saver import ObjectWriteBucket
from ml_flashpoint.core.mlf_logging import get_logger
from ml_flashpoint.core.utils import gc_paused, log_execution_time

_LOGGER = get_logger(__name__)


@log_execution_time(logger=_LOGGER, name="generate_plan", level=logging.INFO)
def generate_plan(
    checkpoint_id: CheckpointContainerId,
    state_dict: torchdistsaver.STATE_DICT_TYPE,
    storage_writer: MemoryStorageWriter,
    planner: torchdistsaver.SavePlanner,
    world_dist_wrapper: _DistWrapper,
    cached_ckpt_structure: tuple[SavePlan, SavePlan, bool] | None = None,
) -> tuple[list[ObjectWriteBucket], torchdistsaver.Metadata | None, SavePlan, SavePlan, bool]:
    """Planning phase of a save.

    Returns ``(write_buckets, global_metadata, central_plan, local_plan, validated_cache_reuse)``.  The last three are
    what the caller keeps as ``cached_ckpt_structure`` for the next save: once the central plan of two consecutive
    saves compares equal, ``validated_cache_reuse`` turns True and later saves skip ``create_local_plan``, the plan
    reduce-scatter and the metadata broadcast (``global_metadata`` is then None: the caller reuses the one it has).
    """
    with gc_paused():  # planning allocates ~10 small objects per tensor; see gc_paused
        return _generate_plan(checkpoint_id, state_dict, storage_writer, planner, world_dist_wrapper, cached_ckpt_structure)


def _generate_plan(checkpoint_id, state_dict, storage_writer, planner, world_dist_wrapper, cached_ckpt_structure):
    cached_central_plan, cached_local_plan, validated = cached_ckpt_structure or (None, None, False)
    global_metadata: torchdistsaver.Metadata | None = None

    def local_step() -> SavePlan:
        planner.set_up_planner(
            state_dict=state_dict,
            storage_meta=storage_writer.storage_meta(),
            is_coordinator=world_dist_wrapper.is_coordinator,
        )
        storage_writer.set_up_storage_writer(world_dist_wrapper.is_coordinator)
        plan = cached_local_plan if (cached_local_plan and validated) else planner.create_local_plan()
        return storage_writer.prepare_local_plan(plan)

    def global_step(all_local_plans: list[SavePlan]) -> list[SavePlan]:
        nonlocal global_metadata
        all_local_plans, global_metadata = planner.create_global_plan(all_local_plans)
        return storage_writer.prepare_global_plan(all_local_plans)

    if validated and cached_central_plan:
        local_plan = local_step()
        central_plan = cached_central_plan
    else:
        with log_execution_time(logger=_LOGGER, name="generate_plan__reduce_scatter_plan"):
            local_plan = local_step()
            central_plan = world_dist_wrapper.reduce_scatter("plan", lambda: local_plan, global_step)
        with log_execution_time(logger=_LOGGER, name="generate_plan__broadcast_metadata"):
            global_metadata = world_dist_wrapper.broadcast_object(global_metadata)

    final_local_plan = planner.finish_plan(central_plan)
    write_buckets = storage_writer.prepare_write_data_buckets(checkpoint_id, final_local_plan, planner)
    return write_buckets, global_metadata, central_plan, local_plan, cached_central_plan == central_plan


@log_execution_time(logger=_LOGGER, name="write_data", level=logging.INFO)
def write_data(
    checkpoint_id: CheckpointContainerId,
    storage_writer: MemoryStorageWriter,
    staged_write_buckets: list[ObjectWriteBucket],
    replicate_after_write: bool,
) -> list[WriteResult]:
    """Write phase; synchronous.  This is the call an async framework runs in its worker."""
    return storage_writer.write_staged_data_buckets(checkpoint_id, staged_write_buckets, replicate_after_write).wait()


@log_execution_time(logger=_LOGGER, name="finish_write", level=logging.INFO)
def finish_write(
    checkpoint_id: CheckpointContainerId,
    storage_writer: MemoryStorageWriter,
    global_metadata: torchdistsaver.Metadata,
    world_dist_wrapper: _DistWrapper,
) -> None:
    """Gathers every rank's write results on the coordinator, broadcasts them, and writes the ``.metadata`` object
    once per node (on node-local rank 0).  Call only after the write of ``checkpoint_id`` is known to be complete."""
    all_results = world_dist_wrapper.gather_object(storage_writer.get_write_results(checkpoint_id))
    with log_execution_time(logger=_LOGGER, name="finish_write__broadcast_results"):
        all_results = world_dist_wrapper.broadcast_object(all_results)
    if torchdist.get_node_local_rank(fallback_rank=0) == 0:
        storage_writer.finish_checkpoint(checkpoint_id=checkpoint_id, metadata=global_metadata, results=all_results)


def _get_local_rank_0_global_ranks() -> list[int]:
    """Global ranks that are rank 0 of their node, assuming every node runs one rank per visible GPU
    (reference: custom_state_dict_saver.py:218-227; nothing calls it there either)."""
    per_node = torch.cuda.device_count()
    return [node * per_node for node in range(utils.get_num_of_nodes())]
