"""Path-shaped identifiers: ``CheckpointContainerId`` names a directory of checkpoint objects,
``CheckpointObjectId`` one object in it.  Both are strings (``UserString``) that have been checked and normalised:
they start with ``/``, carry no trailing slash, and no segment is empty or ends in a dot.  A version container is
called ``step-<N>_ckpt``; the marker of an unfinished one ends in ``_unfinished``.

Class names, methods, rules and messages are those of the reference (src/ml_flashpoint/core/checkpoint_id_types.py
:23-189): savers, loaders, adapters and user code build and compare these ids.
"""

from __future__ import annotations

import abc
import re
from collections import UserString

from ml_flashpoint.core.defaults import DIRTY_MARKER_SUFFIX

_STEP_DIR = re.compile(r"^step-(\d+)_ckpt$")
_STEP_DIR_FORMAT = "step-{step}_ckpt"
_UNFINISHED_STEP_DIR = re.compile(r"^step-(\d+)_ckpt.*_" + re.escape(DIRTY_MARKER_SUFFIX) + r"$")


def _checked(raw: str, type_name: str, leaf: bool) -> str:
    """The normal form of ``raw`` or a ``ValueError`` that says which rule it breaks."""
    if not raw.startswith("/"):
        raise ValueError(f"A {type_name} must begin with '/', got '{raw}' instead.")
    path = raw.rstrip("/")
    if not path:  # nothing but slashes
        if leaf:
            raise ValueError("'/' is not a valid leaf ID.")
        return "/"
    for segment in path[1:].split("/"):
        if not segment:
            raise ValueError(f"Path segment cannot be empty, got '{raw}'")
        if segment.endswith("."):
            raise ValueError(f"Path segment cannot end with a '.', got '{raw}'")
    return path


def _under(parent: "CheckpointContainerId", name: str) -> str:
    if not isinstance(parent, CheckpointContainerId):
        raise TypeError("parent_container_id must be a CheckpointContainerId")
    return f"{parent.data}/{name}"


class CheckpointId(UserString, abc.ABC):
    """Common part of the two kinds of id; instantiate one of the subclasses."""

    @abc.abstractmethod
    def __init__(self, string: str, is_leaf_object: bool):
        super().__init__(_checked(string, type(self).__name__, is_leaf_object))

    def get_parent(self, levels_up: int = 1) -> "CheckpointContainerId | None":
        """The container ``levels_up`` levels above, or None where that would be the root."""
        if levels_up < 1:
            raise ValueError(f"levels_up must be >= 1, got '{levels_up}' instead.")
        kept = self.data.split("/")[1:]
        del kept[len(kept) - min(levels_up, len(kept)):]
        return CheckpointContainerId("/" + "/".join(kept)) if kept else None


class CheckpointContainerId(CheckpointId):
    def __init__(self, string: str):
        super().__init__(string, is_leaf_object=False)
        if self.data == "/":
            raise ValueError("CheckpointContainerId cannot be the root path '/'")

    @staticmethod
    def create_child(parent_container_id: "CheckpointContainerId", child_id: str) -> "CheckpointContainerId":
        """``parent/child``; an empty child (or only slashes) is the parent itself."""
        name = child_id.strip("/")
        joined = _under(parent_container_id, name)
        return CheckpointContainerId(joined) if name else parent_container_id

    # ---- version containers: step-<N>_ckpt ---------------------------------------------------------------------
    @classmethod
    def get_version_container_pattern(cls) -> re.Pattern:
        return _STEP_DIR

    @classmethod
    def get_dirty_version_checkpoint_container_pattern(cls) -> re.Pattern:
        return _UNFINISHED_STEP_DIR

    @classmethod
    def format_version_container(cls, step: int) -> str:
        return _STEP_DIR_FORMAT.format(step=step)

    @classmethod
    def parse_version_container_step(cls, name: str) -> int | None:
        """The step of a well-formed version container name, else None (``TypeError`` for a non-string)."""
        found = _STEP_DIR.match(name)
        return int(found.group(1)) if found else None


class CheckpointObjectId(CheckpointId):
    def __init__(self, string: str):
        super().__init__(string, is_leaf_object=True)

    @staticmethod
    def from_container(parent_container_id: CheckpointContainerId, object_name: str) -> "CheckpointObjectId":
        name = object_name.strip().strip("/")
        joined = _under(parent_container_id, name)
        if not name:
            raise ValueError("object_name must not be empty or consist only of whitespace and slashes")
        return CheckpointObjectId(joined)
