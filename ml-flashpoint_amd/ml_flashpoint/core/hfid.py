"""Human-friendly unique ids, ``<prefix>_<32 hex chars>`` (reference: src/ml_flashpoint/core/hfid.py:19-39)."""

import re
import uuid

_PREFIX_OK = re.compile(r"^[a-z0-9]+$")


def generate_hfid(prefix: str) -> str:
    if not prefix:
        raise ValueError("Prefix cannot be empty.")
    if _PREFIX_OK.match(prefix) is None:
        raise ValueError("Prefix must contain only lowercase alphanumeric characters.")
    return f"{prefix}_{uuid.uuid4().hex}"
