"""Validated, path-shaped identifiers for checkpoint containers (directories) and objects (files).

API, validation rules and messages follow the reference
(src/ml_flashpoint/core/checkpoint_id_types.py:23-189): ids start with ``/``, trailing slashes are dropped,
no segment may be empty or end in ``.``; a container may not be ``/``; version containers are named
``step-<N>_ckpt``.
"""

import abc
import re
from collections import UserString
from typing import Optional

from ml_flashpoint.core.defaults import DIRTY_MARKER_SUFFIX


def _normalise(raw: str, type_name: str, leaf: bool) -> str:
    if not raw.startswith("/"):
        raise ValueError(f"A {type_name} must begin with '/', got '{raw}' instead.")
    path = raw.rstrip("/") or "/"
    if leaf and path == "/":
        raise ValueError(f"'{path}' is not a valid leaf ID.")
    if path != "/":
        for segment in path.split("/")[1:]:
            if segment == "":
                raise ValueError(f"Path segment cannot be empty, got '{raw}'")
            if segment[-1] == ".":
                raise ValueError(f"Path segment cannot end with a '.', got '{raw}'")
    return path


class CheckpointId(UserString, abc.ABC):
    """Base of the two id kinds; use ``CheckpointContainerId`` or ``CheckpointObjectId``."""

    @abc.abstractmethod
    def __init__(self, string: str, is_leaf_object: bool):
        super().__init__(_normalise(string, type(self).__name__, is_leaf_object))

    def get_parent(self, levels_up: int = 1) -> "CheckpointContainerId | None":
        if levels_up < 1:
            raise ValueError(f"levels_up must be >= 1, got '{levels_up}' instead.")
        segments = self.data.split("/")
        if levels_up >= len(segments) - 1:
            return None
        return CheckpointContainerId("/".join(segments[: len(segments) - levels_up]))


class CheckpointContainerId(CheckpointId):
    """A namespace of checkpoint objects (a directory)."""

    _VERSION_CONTAINER_PATTERN = re.compile(r"^step-(\d+)_ckpt$")
    _VERSION_CONTAINER_FORMAT_STRING = "step-{step}_ckpt"
    _DIRTY_VERSION_CONTAINER_PATTERN = re.compile(r"^step-(\d+)_ckpt.*_" + re.escape(DIRTY_MARKER_SUFFIX) + r"$")

    def __init__(self, string: str):
        super().__init__(string, is_leaf_object=False)
        if self.data == "/":
            raise ValueError("CheckpointContainerId cannot be the root path '/'")

    @classmethod
    def get_version_container_pattern(cls) -> re.Pattern:
        return cls._VERSION_CONTAINER_PATTERN

    @classmethod
    def get_dirty_version_checkpoint_container_pattern(cls) -> re.Pattern:
        return cls._DIRTY_VERSION_CONTAINER_PATTERN

    @classmethod
    def format_version_container(cls, step: int) -> str:
        return cls._VERSION_CONTAINER_FORMAT_STRING.format(step=step)

    @classmethod
    def parse_version_container_step(cls, name: str) -> Optional[int]:
        m = cls._VERSION_CONTAINER_PATTERN.match(name)
        return int(m.group(1)) if m else None

    @staticmethod
    def create_child(parent_container_id: "CheckpointContainerId", child_id: str) -> "CheckpointContainerId":
        if not isinstance(parent_container_id, CheckpointContainerId):
            raise TypeError("parent_container_id must be a CheckpointContainerId")
        child = child_id.strip("/")
        if not child:
            return parent_container_id
        return CheckpointContainerId(parent_container_id.data.rstrip("/") + "/" + child)


class CheckpointObjectId(CheckpointId):
    """One checkpoint data blob (a file)."""

    def __init__(self, string: str):
        super().__init__(string, is_leaf_object=True)

    @staticmethod
    def from_container(parent_container_id: CheckpointContainerId, object_name: str) -> "CheckpointObjectId":
        if not isinstance(parent_container_id, CheckpointContainerId):
            raise TypeError("parent_container_id must be a CheckpointContainerId")
        child = object_name.strip().strip("/")
        if not child:
            raise ValueError("object_name must not be empty or consist only of whitespace and slashes")
        return CheckpointObjectId(parent_container_id.data.rstrip("/") + "/" + child)
