"""Recovery discovery: which checkpoint is the newest one every rank can load, and what has to be fetched first.

Host logic only (no GPU work); it follows the reference's algorithm
(src/ml_flashpoint/core/checkpoint_loader.py:221-296 and :340-735):

1. every rank lists the ``step-N_ckpt`` directories under the base that have no ``…_unfinished`` marker beside
   them; the candidates are the *intersection* of the non-empty lists, newest first;
2. for a candidate, every rank lists the objects it holds; the lowest rank that holds ``.metadata`` reads it,
   derives from the object names (``…src<rank>…``) which rank needs which object, adds ``common.pt`` and
   ``.metadata`` for the first rank of every node, and maps every missing object to a rank that has it.  A needed
   object nobody has makes the candidate not viable;
3. the plan is broadcast; an empty plan selects the candidate at once, otherwise every rank fetches its share
   through the replication manager and the candidate is selected if all ranks succeeded.

The collectives are injected (``all_gather_object_func(out_list, obj)``, ``broadcast_object_list_func(list, src=)``)
so the logic runs unchanged in a single process, where they default to trivial stand-ins.

One addition: with ``verify_on_discovery`` an object that has a CRC-32C sidecar is listed only if its bytes still
match it, so a corrupted copy is treated like a missing one (fetched from a peer, or the candidate is skipped).
"""

import fcntl
import os
import re
from collections import defaultdict
from pathlib import Path
from typing import Dict, List, Optional, Set, Tuple

from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.defaults import (
    COMMON_STATE_FNAME,
    DIRTY_MARKER_SUFFIX,
    GLOBAL_RANK_PATTERN,
    default_metadata_object_name,
)
from ml_flashpoint.core.mlf_logging import get_logger
from ml_flashpoint.core.utils import get_num_of_nodes

_LOGGER = get_logger(__name__)

_CONTAINER_PREFIX = re.compile(r"(step-\d+_ckpt)")
RetrievalPlan = Dict[int, List[Tuple[int, str]]]  # target rank -> [(source rank, object path)]


def _single_process_all_gather(out_list: list, obj) -> None:
    out_list[0] = obj


def _single_process_broadcast(obj_list: list, src: int = 0) -> None:
    return None


class CheckpointDiscoveryMixin:
    """Expects the host class to provide ``_global_rank_getter``, ``_local_rank_getter``, ``_world_size_getter``,
    ``_all_gather_object_func``, ``_broadcast_object_list_func``, ``_replication_manager`` and ``read_metadata``."""

    verify_on_discovery: bool = False
    # The reference always requires the Megatron strategy's common-state file on the first rank of every node;
    # set to None for checkpoints written by plain ``dcp.save``, which have no such file.
    common_state_object_name: Optional[str] = COMMON_STATE_FNAME

    def _init_discovery(self) -> None:
        self._available_objects_cache: Dict[CheckpointContainerId, Dict[str, List[int]]] = {}
        if self._all_gather_object_func is None:
            self._all_gather_object_func = _single_process_all_gather
        if self._broadcast_object_list_func is None:
            self._broadcast_object_list_func = _single_process_broadcast

    # ---- hooks ---------------------------------------------------------------------------------------------
    def _get_extra_local_objects(self, container_path: Path) -> List[CheckpointObjectId]:
        """Objects outside the container directory that this rank can offer to others (none by default)."""
        return []

    def _get_extra_needed_objects(self, checkpoint, available_objects_by_rank) -> Set[str]:
        """Objects the first rank of every node needs besides ``common.pt`` and ``.metadata`` (none by default)."""
        return set()

    def _object_is_intact(self, path: str) -> bool:
        """Overridden by loaders that can check an object against its checksum sidecar."""
        return True

    # ---- step 1 ----------------------------------------------------------------------------------------------
    def get_candidate_checkpoints(self, checkpoint_base_container: CheckpointContainerId) -> List[CheckpointContainerId]:
        base = Path(checkpoint_base_container.data)
        mine: List[str] = []
        if base.is_dir():
            finished, unfinished = set(), set()
            for entry in os.listdir(base):
                m = _CONTAINER_PREFIX.match(entry)
                if not m:
                    continue
                if entry.endswith(DIRTY_MARKER_SUFFIX):
                    unfinished.add(m.group(1))  # "step-N_ckpt__<local rank>__unfinished" marks step-N_ckpt
                else:
                    finished.add(entry)
            mine = [str(base / name) for name in finished - unfinished]
        gathered: list = [None] * self._world_size_getter()
        self._all_gather_object_func(gathered, mine)
        lists = [set(paths) for paths in gathered if paths]
        if not lists:
            return []
        common = set.intersection(*lists)
        return sorted(
            (CheckpointContainerId(p) for p in common),
            key=lambda cid: CheckpointContainerId.parse_version_container_step(os.path.basename(cid.data)) or -1,
            reverse=True,
        )

    # ---- step 2 ----------------------------------------------------------------------------------------------
    def get_checkpoint_objects_by_rank(self, checkpoint_container_id: CheckpointContainerId) -> Dict[int, List[CheckpointObjectId]]:
        container = Path(checkpoint_container_id.data)
        mine: List[CheckpointObjectId] = []
        if container.is_dir():
            for entry in os.listdir(container):
                if self.verify_on_discovery and not self._object_is_intact(str(container / entry)):
                    _LOGGER.warning("'%s' does not match its checksum sidecar: treated as missing", container / entry)
                    continue
                mine.append(CheckpointObjectId.from_container(checkpoint_container_id, entry))
            mine.extend(self._get_extra_local_objects(container))
        gathered: list = [None] * self._world_size_getter()
        self._all_gather_object_func(gathered, mine)
        by_rank: Dict[int, List[CheckpointObjectId]] = {}
        locations: Dict[str, List[int]] = defaultdict(list)
        for rank, objects in enumerate(gathered):
            by_rank[rank] = list(objects) if objects else []
            for obj in by_rank[rank]:
                locations[obj.data].append(rank)
        self._available_objects_cache[checkpoint_container_id] = locations
        return by_rank

    def _compute_retrieval_plan(self, checkpoint: CheckpointContainerId,
                                available_objects_by_rank: Dict[int, List[CheckpointObjectId]]) -> Optional[RetrievalPlan]:
        """None: not viable.  Empty: nothing to fetch.  Otherwise target rank -> [(source rank, object path)]."""
        try:
            metadata = self.read_metadata(checkpoint)
        except Exception:
            _LOGGER.warning("Failed to read metadata for '%s'", checkpoint)
            return None
        if metadata.storage_data is None:
            return None
        needed: Dict[int, Set[str]] = defaultdict(set)
        for info in metadata.storage_data.values():
            m = GLOBAL_RANK_PATTERN.search(info.relative_path)
            if m:
                needed[int(m.group(1))].add(str(CheckpointObjectId.from_container(checkpoint, info.relative_path)))
        per_node = {str(CheckpointObjectId.from_container(checkpoint, default_metadata_object_name()))}
        if self.common_state_object_name:
            per_node.add(str(CheckpointObjectId.from_container(checkpoint, self.common_state_object_name)))
        per_node |= set(self._get_extra_needed_objects(checkpoint, available_objects_by_rank))
        world = self._world_size_getter()
        ranks_per_node = world // get_num_of_nodes()
        for rank in range(world):
            if rank % ranks_per_node == 0:
                needed[rank] |= per_node
        holders: Dict[str, List[int]] = defaultdict(list)
        for rank, objects in available_objects_by_rank.items():
            for obj in objects:
                holders[str(obj)].append(rank)
        plan: RetrievalPlan = {}
        for target, wanted in needed.items():
            have = {str(o) for o in available_objects_by_rank.get(target, [])}
            missing = wanted - have
            if not missing:
                continue
            plan[target] = []
            for path in missing:
                sources = holders.get(path)
                if not sources:
                    _LOGGER.warning("Object '%s' is missing globally (needed by rank %s)", path, target)
                    return None
                plan[target].append((sources[0], path))
        return plan

    # ---- step 3 ----------------------------------------------------------------------------------------------
    def retrieve_checkpoint(self, retrieval_plan: RetrievalPlan) -> bool:
        rank = self._global_rank_getter()
        ok = True
        mine = retrieval_plan.get(rank) if retrieval_plan else None
        if mine:
            by_source: Dict[int, List[CheckpointObjectId]] = {}
            for source, path in mine:
                by_source.setdefault(source, []).append(CheckpointObjectId(path))
            for source, objects in by_source.items():
                if not self._replication_manager.sync_bulk_retrieve(
                        source_global_rank=source, object_ids_to_retrieve=objects, container_ids_to_retrieve=[]):
                    _LOGGER.error("Failed to retrieve objects from rank %s", source)
                    ok = False
        outcomes: list = [None] * self._world_size_getter()
        self._all_gather_object_func(outcomes, ok)
        return all(outcomes)

    def get_latest_complete_checkpoint(self, checkpoint_base_container: CheckpointContainerId) -> Optional[CheckpointContainerId]:
        rank = self._global_rank_getter()
        candidates = self.get_candidate_checkpoints(checkpoint_base_container)
        if not candidates:
            _LOGGER.warning("No candidate checkpoints found.")
            return None
        md_name = default_metadata_object_name()
        for checkpoint in candidates:
            by_rank = self.get_checkpoint_objects_by_rank(checkpoint)
            planner_rank = next((r for r in sorted(by_rank)
                                 if any(os.path.basename(o.data) == md_name for o in by_rank[r])), None)
            if planner_rank is None:
                _LOGGER.warning("Rank %s: No metadata found for '%s'", rank, checkpoint)
                continue
            box = [self._compute_retrieval_plan(checkpoint, by_rank) if rank == planner_rank else None]
            self._broadcast_object_list_func(box, src=planner_rank)
            plan = box[0]
            if plan is None:
                _LOGGER.warning("Rank %s: '%s' is not viable", rank, checkpoint)
                continue
            if not plan:
                return checkpoint
            if self.retrieve_checkpoint(plan):
                return checkpoint
            _LOGGER.warning("Failed to retrieve all necessary objects for checkpoint '%s'.", checkpoint)
        _LOGGER.warning("Rank %s: No complete checkpoint found.", rank)
        return None

    # ---- fetch on read -----------------------------------------------------------------------------------------
    def _try_retrieve_object_if_missing(self, checkpoint_object_id: CheckpointObjectId) -> bool:
        """A missing object is fetched from the first rank that listed it during discovery; a lock file keeps
        the ranks of one node from fetching the same object twice."""
        if os.path.exists(checkpoint_object_id.data):
            return True
        if not self._replication_manager:
            _LOGGER.error("ReplicationManager is not initialized.")
            return False
        sources = self._available_objects_cache.get(checkpoint_object_id.get_parent(), {}).get(checkpoint_object_id.data)
        if not sources:
            return False
        try:
            with open(f"{checkpoint_object_id.data}.lock", "w") as lock_file:
                fcntl.flock(lock_file, fcntl.LOCK_EX)
                try:
                    if os.path.exists(checkpoint_object_id.data):
                        return True
                    return bool(self._replication_manager.sync_bulk_retrieve(
                        source_global_rank=sources[0], object_ids_to_retrieve=[checkpoint_object_id],
                        container_ids_to_retrieve=[]))
                finally:
                    fcntl.flock(lock_file, fcntl.LOCK_UN)
        except Exception:
            _LOGGER.exception("Error during retrieval/locking for '%s'", checkpoint_object_id.data)
            return False
