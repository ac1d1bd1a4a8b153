"""Constants of the on-buffer format and of checkpoint naming.

Values follow the reference (src/ml_flashpoint/core/defaults.py:18-36); they are part of the wire format and
must not change.
"""

import enum
import re

DIRTY_MARKER_SUFFIX = "unfinished"
GLOBAL_RANK_PATTERN = re.compile(r"src(\d+)")
COMMON_STATE_FNAME = "common.pt"


class CheckpointFormat(bytes, enum.Enum):
    """8-byte signature stored at offset 8 of a buffer's metadata block."""

    TORCH_SAVE = b"TORCH___"  # records are torch.save streams
    MLF_FORMAT = b"MLF_TENS"  # records are <u32 len><pickled TensorHeader><raw bytes>


def default_metadata_object_name() -> str:
    return ".metadata"
