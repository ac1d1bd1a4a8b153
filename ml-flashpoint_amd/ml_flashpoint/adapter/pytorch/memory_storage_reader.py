"""PyTorch DCP ``StorageReader`` that loads from in-memory buffer objects through a checkpoint loader plug-in
(reference: src/ml_flashpoint/adapter/pytorch/memory_storage_reader.py:46-160)."""

import logging
import os
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import Dict, List, Union

import torch
from torch.distributed.checkpoint import StorageReader
from torch.distributed.checkpoint import metadata as torchdistmeta
from torch.distributed.checkpoint.filesystem import FileSystem, _StorageInfo
from torch.distributed.checkpoint.planner import LoadPlan, LoadPlanner, ReadItem
from torch.futures import Future
from typing_extensions import override

from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_loader import MLFlashpointCheckpointLoader
from ml_flashpoint.core.hfid import generate_hfid
from ml_flashpoint.core.mlf_logging import get_logger
from ml_flashpoint.core.utils import log_execution_time

_LOGGER = get_logger(__name__)


class MemoryStorageReader(StorageReader):
    _path: str
    _checkpoint_container_id: CheckpointContainerId
    _load_id: str
    _checkpoint_loader: MLFlashpointCheckpointLoader
    _storage_data: dict[torchdistmeta.MetadataIndex, _StorageInfo] | None

    def __init__(self, path: Union[str, os.PathLike], checkpoint_loader: MLFlashpointCheckpointLoader):
        super().__init__()
        self.reset(path)
        self._checkpoint_loader = checkpoint_loader
        self._storage_data = None

    @override
    def reset(self, checkpoint_id: Union[str, os.PathLike, None] = None) -> None:
        self._path = checkpoint_id
        self._checkpoint_container_id = CheckpointContainerId(str(checkpoint_id))
        self._load_id = generate_hfid("memreaderload")

    @override
    @log_execution_time(logger=_LOGGER, name="read_metadata", level=logging.INFO)
    def read_metadata(self) -> torchdistmeta.Metadata:
        metadata = self._checkpoint_loader.read_metadata(self._checkpoint_container_id)
        if self._load_id:
            metadata.storage_meta.load_id = self._load_id
        return metadata

    @override
    def set_up_storage_reader(self, metadata: torchdistmeta.Metadata, is_coordinator: bool) -> None:
        self._storage_data = metadata.storage_data
        if self._storage_data is None:
            raise ValueError("metadata.storage_data cannot be None.")

    @override
    def prepare_local_plan(self, plan: LoadPlan) -> LoadPlan:
        return plan

    @override
    def prepare_global_plan(self, plans: list[LoadPlan]) -> list[LoadPlan]:
        return plans

    @override
    @log_execution_time(logger=_LOGGER, name="read_data", level=logging.INFO)
    def read_data(self, plan: LoadPlan, planner: LoadPlanner) -> Future[None]:
        """One ``loader.read_data`` task per object file, run on a thread pool; exceptions propagate."""
        per_file: Dict[str, List[ReadItem]] = {}
        for item in plan.items:
            per_file.setdefault(self._storage_data[item.storage_index].relative_path, []).append(item)
        if per_file:
            start = time.perf_counter()
            with ThreadPoolExecutor() as pool:
                tasks = [
                    pool.submit(
                        self._checkpoint_loader.read_data,
                        CheckpointObjectId(str(Path(self._path) / relative_path)),
                        items,
                        planner,
                        self._storage_data,
                    )
                    for relative_path, items in per_file.items()
                ]
                for task in tasks:
                    task.result()
            duration = time.perf_counter() - start
            total = sum(self._storage_data[item.storage_index].length for item in plan.items)
            if duration > 0:
                _LOGGER.info(
                    "Read %d bytes in %.4f s (%.2f GB/s) from %d files",
                    total,
                    duration,
                    (total / 1e9) / duration,
                    len(per_file),
                )
        else:
            # a single-process load has no process group to ask; the line is informational either way
            rank = torch.distributed.get_rank() if torch.distributed.is_initialized() else 0
            _LOGGER.info("Rank %d: No files to read for plan in '%s'", rank, self._path)
        done: Future = Future()
        done.set_result(None)
        return done

    @classmethod
    @override
    def validate_checkpoint_id(cls, checkpoint_id: Union[str, os.PathLike]) -> bool:
        return FileSystem.validate_checkpoint_id(checkpoint_id)
