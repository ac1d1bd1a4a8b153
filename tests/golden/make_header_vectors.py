"""Writes tests/golden/tensor_header_vectors.json: (dtype, shape) -> hex of the reference's record header.

Run once, in the development container only, where the reference checkout is mounted:

    python tests/golden/make_header_vectors.py /root/reference/src

It imports exactly one leaf module of the reference, ``ml_flashpoint.core.tensor_header`` (pure Python, depends
on torch only), calls ``TensorHeader(dtype, shape).to_bytes()`` for a fixed list of cases and stores the bytes.
The exact header bytes are the one part of the format that no test, fixture or closed form in the reference
pins, hence these vectors.  The JSON is data; nothing of the reference's source is stored.
"""

import json
import os
import sys


def main() -> None:
    ref_src = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/src"
    sys.path.insert(0, ref_src)
    import torch
    from ml_flashpoint.core.tensor_header import TensorHeader  # the reference's class

    assert TensorHeader.__module__ == "ml_flashpoint.core.tensor_header"
    assert os.path.abspath(sys.modules[TensorHeader.__module__].__file__).startswith(os.path.abspath(ref_src))

    cases = [
        ("float32", []),
        ("float32", [0]),
        ("float32", [2, 2]),
        ("float32", [768]),
        ("float32", [50257, 768]),
        ("bfloat16", [4096, 14336]),
        ("bfloat16", [128256, 4096]),
        ("float16", [3, 5, 7]),
        ("float64", [1]),
        ("int64", [255]),
        ("int64", [256]),
        ("int64", [65535]),
        ("int64", [65536]),
        ("int32", [2147483647]),
        ("int32", [2147483648]),
        ("int16", [1, 1, 1, 1, 1]),
        ("int8", [4, 0, 3]),
        ("uint8", [1024]),
        ("bool", [17]),
        ("float8_e4m3fn", [1024, 16384]),
        ("float8_e5m2", [16, 16]),
        ("complex64", [2, 3]),
        ("float32", [1, 2, 3, 4, 5, 6, 7, 8]),
        ("float32", [300, 70000, 2]),
    ]
    out = []
    for dtype_name, shape in cases:
        raw = TensorHeader(dtype=getattr(torch, dtype_name), shape=torch.Size(shape)).to_bytes()
        out.append({"dtype": dtype_name, "shape": shape, "hex": raw.hex()})
    dest = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tensor_header_vectors.json")
    with open(dest, "w") as f:
        json.dump({"python": sys.version.split()[0], "torch": torch.__version__, "vectors": out}, f, indent=1)
    print(f"wrote {len(out)} vectors to {dest}")


if __name__ == "__main__":
    main()
