"""Loader plug-in interface of the restore path (reference: src/ml_flashpoint/core/checkpoint_loader.py:57-118).

The implementation shipped here is ``HipMLFlashpointCheckpointLoader`` (ml_flashpoint/hip/checkpoint_loader.py),
also reachable under the reference's class name ``DefaultMLFlashpointCheckpointLoader`` from this module.
"""

import abc
from typing import List, Optional

from torch.distributed.checkpoint import Metadata
from torch.distributed.checkpoint.filesystem import _StorageInfo
from torch.distributed.checkpoint.planner import LoadPlanner, ReadItem

from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.defaults import default_metadata_object_name


class MLFlashpointCheckpointLoader(abc.ABC):
    @abc.abstractmethod
    def read_metadata(
        self,
        checkpoint_id: CheckpointContainerId,
        object_name: str = default_metadata_object_name(),
    ) -> Metadata:
        """Returns the ``Metadata`` stored at ``<checkpoint_id>/<object_name>``."""

    @abc.abstractmethod
    def read_data(
        self,
        checkpoint_object_id: CheckpointObjectId,
        read_items: List[ReadItem],
        planner: LoadPlanner,
        storage_data: dict[int, _StorageInfo],
    ) -> None:
        """Loads every item of ``read_items`` that lives in ``checkpoint_object_id`` into the planner's targets."""

    @abc.abstractmethod
    def get_latest_complete_checkpoint(
        self, checkpoint_base_container: CheckpointContainerId
    ) -> Optional[CheckpointContainerId]:
        """Newest ``step-N_ckpt`` under the base container that has no unfinished marker, or None."""


def __getattr__(name):
    if name == "DefaultMLFlashpointCheckpointLoader":
        from ml_flashpoint.hip.checkpoint_loader import HipMLFlashpointCheckpointLoader

        return HipMLFlashpointCheckpointLoader
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
