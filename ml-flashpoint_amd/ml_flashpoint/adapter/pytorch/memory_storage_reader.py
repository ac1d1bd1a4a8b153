"""DCP ``StorageReader`` over checkpoint buffer objects: sorts a load plan by object file and hands each file's
requests to a loader plug-in (same public surface as the reference's adapter,
src/ml_flashpoint/adapter/pytorch/memory_storage_reader.py:46-160).

With the gfx950 loader one object is one pipelined transfer (file -> pinned slots -> HBM image -> unpack kernels into
the planner's targets), so all requests of a file have to arrive in one call; files are independent and run on
separate threads.
"""

from __future__ import annotations

import collections
import concurrent.futures
import logging
import os
import time

import torch.distributed as torchdist
from torch.distributed.checkpoint.filesystem import FileSystem
from torch.distributed.checkpoint.metadata import Metadata
from torch.distributed.checkpoint.planner import LoadPlan, LoadPlanner
from torch.distributed.checkpoint.storage import StorageReader
from torch.futures import Future
from typing_extensions import override

from ml_flashpoint.core import utils
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_loader import MLFlashpointCheckpointLoader
from ml_flashpoint.core.hfid import generate_hfid
from ml_flashpoint.core.mlf_logging import get_logger

_LOGGER = get_logger(__name__)


class MemoryStorageReader(StorageReader):
    def __init__(self, path: str | os.PathLike, checkpoint_loader: MLFlashpointCheckpointLoader):
        super().__init__()
        self._checkpoint_loader = checkpoint_loader
        self._storage_data = None  # MetadataIndex -> _StorageInfo, known once the metadata has been read
        self.reset(path)

    @override
    def reset(self, checkpoint_id: str | os.PathLike | None = None) -> None:
        """Points the reader at another checkpoint; every (re)start of a load gets its own load id."""
        self._path = checkpoint_id
        self._checkpoint_container_id = CheckpointContainerId(str(checkpoint_id))
        self._load_id = generate_hfid("memreaderload")

    @classmethod
    @override
    def validate_checkpoint_id(cls, checkpoint_id: str | os.PathLike) -> bool:
        return FileSystem.validate_checkpoint_id(checkpoint_id)

    @override
    @utils.log_execution_time(logger=_LOGGER, name="read_metadata", level=logging.INFO)
    def read_metadata(self) -> Metadata:
        metadata = self._checkpoint_loader.read_metadata(self._checkpoint_container_id)
        if self._load_id:
            metadata.storage_meta.load_id = self._load_id
        return metadata

    @override
    def set_up_storage_reader(self, metadata: Metadata, is_coordinator: bool) -> None:
        if metadata.storage_data is None:
            self._storage_data = None
            raise ValueError("metadata.storage_data cannot be None.")
        self._storage_data = metadata.storage_data

    @override
    def prepare_local_plan(self, plan: LoadPlan) -> LoadPlan:
        return plan

    @override
    def prepare_global_plan(self, plans: list[LoadPlan]) -> list[LoadPlan]:
        return plans

    @override
    @utils.log_execution_time(logger=_LOGGER, name="read_data", level=logging.INFO)
    def read_data(self, plan: LoadPlan, planner: LoadPlanner) -> Future[None]:
        """Blocking; the returned future is already complete.  The first failing file's exception is raised."""
        where = self._storage_data
        by_file = collections.defaultdict(list)  # relative path -> requests, in plan order
        for request in plan.items:
            by_file[where[request.storage_index].relative_path].append(request)
        if by_file:
            began = time.perf_counter()
            root = os.fspath(self._path)
            with concurrent.futures.ThreadPoolExecutor() as pool:
                running = [
                    pool.submit(self._checkpoint_loader.read_data, CheckpointObjectId(os.path.join(root, name)),
                                requests, planner, where)
                    for name, requests in by_file.items()
                ]
                for task in running:
                    task.result()
            utils.log_rate(_LOGGER, "Read", sum(where[r.storage_index].length for r in plan.items),
                           time.perf_counter() - began, len(by_file), "files")
        else:
            # a single-process load has no process group to ask; the line is informational either way
            rank = torchdist.get_rank() if torchdist.is_initialized() else 0
            _LOGGER.info("Rank %d: No files to read for plan in '%s'", rank, self._path)
        finished: Future = Future()
        finished.set_result(None)
        return finished
