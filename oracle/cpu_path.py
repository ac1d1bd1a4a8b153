"""CPU oracle, part 3: the reference's CPU save/restore path as plug-ins, restated.

TEST INFRASTRUCTURE ONLY (checker and CPU baseline).  The shipped package never imports this module.

``OracleCheckpointSaver`` / ``OracleCheckpointLoader`` do what the reference's default saver/loader do, step by step,
on the host, with plain ``mmap`` files instead of the package's buffer layer:

* ``stage_data``          - core/checkpoint_saver.py:347-360 (per-tensor ``.to("cpu")`` + one device synchronize)
* ``prepare_write_data``  - core/checkpoint_saver.py:364-431 (torch's ``_split_by_size_and_type``; CPU views are
                            cloned and made contiguous; object names ``<prefix>_<k>_src<rank>.distcp``)
* ``write_data``          - core/checkpoint_saver.py:435-519,622-707,764-800 (thread-count rule for torch intra-op
                            threads; per tensor: header, then ``torch.frombuffer(slice).reshape().copy_(tensor)``;
                            byte blobs after the tensors; offsets relative to the data section)
* ``read_data``           - core/checkpoint_loader.py:300-336 with ``read_tensor`` :177-219 (copy the record out of
                            the mapping, ``frombuffer``, narrow, ``target.copy_``)

They implement the package's abstract plug-in interfaces only so that the same adapters can drive either side in
tests; no data-moving code of the package is used.  The byte format comes from ``oracle/mlf_format.py``.
"""

import io
import mmap
import os
import pickle
from typing import List, Optional

import torch
from torch.distributed.checkpoint.filesystem import _split_by_size_and_type, _StorageInfo
from torch.distributed.checkpoint.planner import LoadItemType, WriteItemType
from torch.distributed.checkpoint.storage import WriteResult

from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_loader import MLFlashpointCheckpointLoader
from ml_flashpoint.core.checkpoint_saver import MLFlashpointCheckpointSaver, ObjectWriteBucket

from . import mlf_format as fmt


def write_object(path: str, tensors, blobs, capacity: int):
    """Writes one object file the reference's way and returns [(offset, length)] per item.

    ``capacity`` plays the role of ``initial_buffer_size_bytes``: the file is created at ``capacity + 4096`` bytes,
    mapped, filled, and truncated to ``4096 + written`` at the end.
    """
    os.makedirs(os.path.dirname(path), exist_ok=True)
    if os.path.lexists(path):
        os.remove(path)
    total = capacity + fmt.METADATA_SIZE
    fd = os.open(path, os.O_CREAT | os.O_RDWR | os.O_TRUNC, 0o666)
    try:
        os.ftruncate(fd, total)
        mm = mmap.mmap(fd, total, mmap.MAP_SHARED, mmap.PROT_READ | mmap.PROT_WRITE)
        mv = memoryview(mm)
        pos = 0
        spans = []
        try:
            for t in tensors:
                start = pos
                hdr = fmt.header_bytes(fmt.dtype_name(t.dtype), tuple(t.shape))
                if fmt.METADATA_SIZE + pos + len(hdr) > total:
                    raise ValueError("Write operation exceeds buffer capacity.")
                mv[fmt.METADATA_SIZE + pos : fmt.METADATA_SIZE + pos + len(hdr)] = hdr
                pos += len(hdr)
                nbytes = t.numel() * t.element_size()
                if nbytes:
                    if fmt.METADATA_SIZE + pos + nbytes > total:
                        raise ValueError("Requested slice exceeds buffer capacity")
                    dest = mv[fmt.METADATA_SIZE + pos : fmt.METADATA_SIZE + pos + nbytes]
                    torch.frombuffer(dest, dtype=t.dtype, count=t.numel()).reshape(t.shape).copy_(t)
                    del dest
                    pos += nbytes
                spans.append((start, pos - start))
            for blob in blobs:
                if fmt.METADATA_SIZE + pos + len(blob) > total:
                    raise ValueError("Write operation exceeds buffer capacity.")
                mv[fmt.METADATA_SIZE + pos : fmt.METADATA_SIZE + pos + len(blob)] = blob
                spans.append((pos, len(blob)))
                pos += len(blob)
            mv[: fmt.METADATA_SIZE] = fmt.metadata_block(pos, fmt.SIGNATURE_MLF)
        finally:
            mv.release()
            mm.close()
        os.ftruncate(fd, fmt.METADATA_SIZE + pos)
    finally:
        os.close(fd)
    return spans


def _zero() -> int:
    return 0


def _no_barrier() -> None:
    return None


class OracleCheckpointSaver(MLFlashpointCheckpointSaver):
    def __init__(self, global_rank_getter=_zero, local_rank_getter=_zero, global_barrier_func=_no_barrier,
                 initial_buffer_size_bytes: int = 1 << 30, accelerator_count: Optional[int] = None):
        self._global_rank_getter = global_rank_getter
        self._local_rank_getter = local_rank_getter
        self._barrier_func = global_barrier_func
        self._initial_buffer_size_bytes = initial_buffer_size_bytes
        self._accelerator_count = accelerator_count

    def initialize_checkpoint(self, checkpoint_id: CheckpointContainerId) -> None:
        marker = f"{str(checkpoint_id).rstrip('/')}__{self._local_rank_getter()}__unfinished"
        os.makedirs(os.path.dirname(marker), exist_ok=True)
        open(marker, "w").close()
        os.makedirs(checkpoint_id.data, exist_ok=True)

    def stage_data(self, checkpoint_id, state_dict: dict, non_blocking: bool = True) -> dict:
        staged = {k: (v.to(device="cpu", non_blocking=non_blocking) if isinstance(v, torch.Tensor) else v)
                  for k, v in state_dict.items()}
        if non_blocking and torch.cuda.is_available():
            torch.cuda.synchronize()
        return staged

    def prepare_write_data(self, checkpoint_id, write_items, write_item_resolver, object_name_prefix, bucket_count):
        def clone_if_needed(t: torch.Tensor):
            if t.device.type != "cpu":
                return t
            is_view = t.untyped_storage().size() != t.numel() * t.itemsize
            return (t.clone() if is_view else t).contiguous()

        buckets = []
        for group in _split_by_size_and_type(max(bucket_count, 1), write_items):
            if not group:
                continue
            blobs = [(i, write_item_resolver.resolve_data(i)) for i in group if i.type == WriteItemType.BYTE_IO]
            tensors = [(i, clone_if_needed(write_item_resolver.resolve_data(i).detach()))
                       for i in group if i.type != WriteItemType.BYTE_IO]
            if blobs or tensors:
                name = f"{object_name_prefix}_{len(buckets)}_src{self._global_rank_getter()}.distcp"
                buckets.append(ObjectWriteBucket(CheckpointObjectId.from_container(checkpoint_id, name), name, blobs, tensors))
        return buckets

    def torch_thread_count(self, thread_count: int = 1) -> int:
        ranks = self._accelerator_count if self._accelerator_count is not None else torch.cuda.device_count()
        return max(1, (os.cpu_count() or 1) // 2 // max(ranks, 1) // max(thread_count, 1))

    def write_data(self, checkpoint_id, write_buckets, replicate_after_write=False, thread_count: int = 1):
        original = torch.get_num_threads()
        torch.set_num_threads(self.torch_thread_count(thread_count))
        try:
            results: List[WriteResult] = []
            for bucket in write_buckets:
                blobs = []
                for _, data in bucket.bytesio_data:
                    data.seek(0)
                    blobs.append(data.read())
                spans = write_object(bucket.object_id.data, [t for _, t in bucket.tensor_data], blobs,
                                     self._initial_buffer_size_bytes)
                items = [i for i, _ in bucket.tensor_data] + [i for i, _ in bucket.bytesio_data]
                results.extend(
                    WriteResult(index=i.index, size_in_bytes=length,
                                storage_data=_StorageInfo(relative_path=bucket.object_name, offset=off, length=length))
                    for i, (off, length) in zip(items, spans)
                )
            return results
        finally:
            torch.set_num_threads(original)

    def write_metadata(self, checkpoint_id, metadata, md_object_name: str = ".metadata"):
        path = os.path.join(checkpoint_id.data, md_object_name)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path + ".tmp", "wb") as f:
            pickle.dump(metadata, f)
        os.rename(path + ".tmp", path)

    def finalize_checkpoint(self, checkpoint_id):
        marker = f"{str(checkpoint_id).rstrip('/')}__{self._local_rank_getter()}__unfinished"
        if os.path.exists(marker):
            os.remove(marker)
        self._barrier_func()
        return None


class OracleCheckpointLoader(MLFlashpointCheckpointLoader):
    def read_metadata(self, checkpoint_id, object_name: str = ".metadata"):
        with open(os.path.join(checkpoint_id.data, object_name), "rb") as f:
            return pickle.load(f)

    def read_data(self, checkpoint_object_id, read_items, planner, storage_data) -> None:
        path = checkpoint_object_id.data
        if not os.path.exists(path):
            raise FileNotFoundError(f"Checkpoint object '{path}' does not exist on any node in the cluster")
        with open(path, "rb") as f:
            mm = mmap.mmap(f.fileno(), 0, mmap.MAP_SHARED, mmap.PROT_READ)
            try:
                assert mm[8:16] == fmt.SIGNATURE_MLF, "oracle loader restates the MLF_TENS branch only"
                for req in read_items:
                    md = storage_data[req.storage_index]
                    begin = fmt.METADATA_SIZE + md.offset
                    record = mm[begin : begin + md.length]  # the copy BufferIO.read() makes
                    if req.type == LoadItemType.BYTE_IO:
                        planner.load_bytes(req, io.BytesIO(record))
                        continue
                    tensor = fmt.read_item(record, req.storage_offsets, req.lengths)
                    target = planner.resolve_tensor(req).detach()
                    assert target.size() == tensor.size(), (
                        f"req {req.storage_index} mismatch sizes {target.size()} vs {tensor.size()}")
                    target.copy_(tensor)
                    planner.commit_tensor(req, target)
            finally:
                mm.close()

    def get_latest_complete_checkpoint(self, checkpoint_base_container):
        return None
