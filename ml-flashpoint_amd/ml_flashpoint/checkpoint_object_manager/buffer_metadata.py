"""The 4096-byte metadata block at offset 0 of every buffer file.

Little-endian, packed: ``u64 len_written_data`` @0, ``char[8] format_signature`` @8, 4080 reserved zero bytes
(reference: src/ml_flashpoint/checkpoint_object_manager/buffer_metadata.py:18-44).
"""

import ctypes

METADATA_SIZE = 4096


class BufferMetadataType(ctypes.LittleEndianStructure):
    _pack_ = 1
    _fields_ = [
        ("len_written_data", ctypes.c_uint64),
        ("format_signature", ctypes.c_char * 8),
        ("reserved", ctypes.c_uint8 * (METADATA_SIZE - 16)),
    ]


assert ctypes.sizeof(BufferMetadataType) == METADATA_SIZE


def get_metadata_str(metadata: "BufferMetadataType | None") -> str:
    if metadata is None:
        return "[Metadata: None]"
    return f"Metadata(len_written_data={metadata.len_written_data})"
