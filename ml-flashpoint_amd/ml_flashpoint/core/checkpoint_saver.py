"""Saver plug-in interface of the save path, and the types that cross it.

``MLFlashpointCheckpointSaver`` is the seam the framework adapters call; the method names, argument meaning and
call order are the reference's (src/ml_flashpoint/core/checkpoint_saver.py:106-286):

  Megatron-style   initialize_checkpoint -> prepare_write_data -> [stage] -> write_data -> write_metadata
                   -> finalize_checkpoint
  PyTorch DCP      initialize_checkpoint -> (stage_data) -> write_data -> write_metadata -> finalize_checkpoint

The implementation shipped here is ``HipMLFlashpointCheckpointSaver`` (ml_flashpoint/hip/checkpoint_saver.py),
also reachable under the reference's class name ``DefaultMLFlashpointCheckpointSaver`` from this module.
"""

import abc
import concurrent.futures
import dataclasses
import io
import subprocess
from typing import Protocol, Union

import torch
from torch.distributed.checkpoint import metadata as torchdistmeta
from torch.distributed.checkpoint.planner import WriteItem
from torch.distributed.checkpoint.storage import WriteResult

from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.defaults import default_metadata_object_name

DEFAULT_INITIAL_BUFFER_SIZE_BYTES = 16 * 1024 * 1024 * 1024
"""Default capacity of a standalone (non-pooled) buffer: 16 GiB."""

_DEFAULT_OBJ_NAME_SUFFIX = ".distcp"


@dataclasses.dataclass
class ObjectWriteBucket:
    """Everything that goes into one checkpoint object (one file)."""

    object_id: CheckpointObjectId
    object_name: str
    bytesio_data: list[tuple[WriteItem, io.BytesIO]]
    tensor_data: list[tuple[WriteItem, torch.Tensor]]


class WriteItemResolver(Protocol):
    """Anything with ``resolve_data`` - a DCP ``SavePlanner`` as is, or a custom lookup into a state dict."""

    @abc.abstractmethod
    def resolve_data(self, write_item: WriteItem) -> Union[torch.Tensor, io.BytesIO]:
        """Returns the tensor (any device, any strides, may be a view) or the serialized bytes of ``write_item``.
        Must be idempotent and thread-safe."""


class MLFlashpointCheckpointSaver(abc.ABC):
    @abc.abstractmethod
    def initialize_checkpoint(self, checkpoint_id: CheckpointContainerId) -> None:
        """Marks ``checkpoint_id`` as in progress (dirty marker) before anything else is created for it."""

    @abc.abstractmethod
    def stage_data(self, checkpoint_id: CheckpointContainerId, state_dict: dict, non_blocking: bool = True) -> dict:
        """Returns a flat state dict whose tensors are host-resident copies.  Blocking: done when it returns."""

    @abc.abstractmethod
    def prepare_write_data(
        self,
        checkpoint_id: CheckpointContainerId,
        write_items: list[WriteItem],
        write_item_resolver: WriteItemResolver,
        object_name_prefix: str,
        bucket_count: int,
    ) -> list[ObjectWriteBucket]:
        """Resolves the items and groups them into at most ``bucket_count`` objects."""

    @abc.abstractmethod
    def write_data(
        self,
        checkpoint_id: CheckpointContainerId,
        write_buckets: list[ObjectWriteBucket],
        thread_count: int,
        replicate_after_write: bool,
    ) -> list[WriteResult]:
        """Writes every bucket into its buffer object; synchronous.  Returns one WriteResult per item."""

    def async_replicate_object(self, object_id: CheckpointObjectId) -> list[concurrent.futures.Future]:
        """Starts replication of a written object to peer nodes."""

    @abc.abstractmethod
    def write_metadata(
        self,
        checkpoint_id: CheckpointContainerId,
        metadata: torchdistmeta.Metadata,
        md_object_name: str = default_metadata_object_name(),
    ):
        """Atomically writes ``<checkpoint_id>/<md_object_name>``."""

    @abc.abstractmethod
    def finalize_checkpoint(self, checkpoint_id: CheckpointContainerId) -> Union[subprocess.Popen, None]:
        """Removes the dirty marker, waits on the global barrier, and (local rank 0) deletes older steps in the
        background; returns that process or None."""


def __getattr__(name):
    # The reference's concrete class name resolves to the gfx950 implementation (lazy: avoids an import cycle).
    if name == "DefaultMLFlashpointCheckpointSaver":
        from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver

        return HipMLFlashpointCheckpointSaver
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
