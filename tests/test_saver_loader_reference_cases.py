"""The reference's own saver and loader test cases (tests/core/test_checkpoint_saver.py:145-187, :274-322, :858-1050,
:1151-1700, :1760-1867; tests/core/test_checkpoint_loader.py:160-203, :223-380, :542-728), restated and run against
two implementations of the plug-in interfaces:

* ``oracle`` - the CPU restatement under ``oracle/`` (runs everywhere; this is what pins the checker itself to the
  expectations the reference's tests hold), and
* ``hip``    - the gfx950 saver/loader with the same inputs resident in HBM (GPU only).

Records are taken apart here with ``struct`` + ``pickle`` + ``numpy`` only, so the check shares no code with either
writer.
"""

import io
import os
import pickle
import struct

import numpy as np
import pytest
import torch
import torch.distributed.checkpoint.metadata as torchdistmeta
from torch.distributed.checkpoint.filesystem import _StorageInfo
from torch.distributed.checkpoint.metadata import MetadataIndex
from torch.distributed.checkpoint.planner import (
    BytesIOWriteData,
    LoadItemType,
    ReadItem,
    TensorWriteData,
    WriteItem,
    WriteItemType,
)

from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.tensor_header import TensorHeader
from oracle.cpu_path import OracleCheckpointLoader, OracleCheckpointSaver

GPU = pytest.mark.gpu
BACKENDS = ["oracle", pytest.param("hip", marks=GPU)]


class _Replication:
    """Stands in for the replication manager: records what it is handed."""

    def __init__(self):
        self.calls = []

    def async_replicate(self, buffer_io):
        self.calls.append(buffer_io)
        return []


class _Backend:
    def __init__(self, name):
        self.name = name
        self.replication = _Replication()
        if name == "oracle":
            self.device = "cpu"
            self.saver = OracleCheckpointSaver(initial_buffer_size_bytes=1 << 20)
            self.loader = OracleCheckpointLoader()
        else:
            from ml_flashpoint.hip.checkpoint_loader import HipMLFlashpointCheckpointLoader
            from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver

            self.device = "cuda:0"
            self.saver = HipMLFlashpointCheckpointSaver(
                global_rank_getter=lambda: 0,
                local_rank_getter=lambda: 0,
                global_barrier_func=lambda: None,
                ckpt_obj_manager=CheckpointObjectManager(),
                replication_manager=self.replication,
                initial_buffer_size_bytes=1 << 20,
            )
            self.loader = HipMLFlashpointCheckpointLoader(CheckpointObjectManager(), None)

    def put(self, value):
        return value.to(self.device) if isinstance(value, torch.Tensor) else value


@pytest.fixture(params=BACKENDS)
def backend(request):
    CheckpointObjectManager._worker_pool = None
    yield _Backend(request.param)
    CheckpointObjectManager().teardown_pool()


class _Resolver:
    def __init__(self, data_map):
        self.data_map = data_map

    def resolve_data(self, write_item):
        if write_item.index in self.data_map:
            return self.data_map[write_item.index]
        raise KeyError(f"Index {write_item.index} not found in data map")


def _tensor_item(fqn, tensor):
    return WriteItem(
        index=MetadataIndex(fqn=fqn),
        type=WriteItemType.TENSOR,
        tensor_data=TensorWriteData(chunk=None, properties=torchdistmeta.TensorProperties(dtype=tensor.dtype), size=tensor.shape),
    )


def _bytes_item(fqn, raw):
    return WriteItem(index=MetadataIndex(fqn=fqn), type=WriteItemType.BYTE_IO, bytes_io_data=BytesIOWriteData(len(raw)))


def _plan(backend, entries):
    """entries: {fqn: tensor or bytes} -> (write items, resolver over inputs placed where the backend wants them)."""
    items, data_map = [], {}
    for fqn, value in entries.items():
        if isinstance(value, torch.Tensor):
            items.append(_tensor_item(fqn, value))
            data_map[MetadataIndex(fqn=fqn)] = backend.put(value)
        else:
            items.append(_bytes_item(fqn, value))
            data_map[MetadataIndex(fqn=fqn)] = io.BytesIO(value)
    return items, _Resolver(data_map)


_NUMPY_OF = {torch.bfloat16: np.uint16, torch.float16: np.float16, torch.float32: np.float32, torch.int32: np.int32,
             torch.int64: np.int64}


def _raw(tensor):
    if tensor.dtype == torch.bfloat16:
        return tensor.contiguous().view(torch.int16).numpy().tobytes()
    return tensor.contiguous().numpy().tobytes()


def _parse_record(record: bytes):
    """[u32 length][pickled header][raw bytes] -> (dtype, shape, payload bytes)."""
    (header_len,) = struct.unpack("<I", record[:4])
    header = pickle.loads(record[4 : 4 + header_len])
    assert isinstance(header, TensorHeader)
    return header.dtype, header.shape, record[4 + header_len :]


def _assert_tensor_record(path, offset, length, expected):
    with open(path, "rb") as f:
        f.seek(METADATA_SIZE + offset)
        record = f.read(length)
    assert len(record) == length
    dtype, shape, payload = _parse_record(record)
    assert dtype == expected.dtype and shape == expected.shape and isinstance(shape, torch.Size)
    assert payload == _raw(expected)                       # C-contiguous little-endian bytes, nothing else
    if expected.numel():
        back = torch.from_numpy(np.frombuffer(payload, dtype=_NUMPY_OF[expected.dtype]).copy())
        back = back.view(expected.dtype) if expected.dtype == torch.bfloat16 else back
        assert torch.equal(back.reshape(expected.shape), expected)


def _save(backend, cid, entries, bucket_count=1, thread_count=None, replicate=False):
    items, resolver = _plan(backend, entries)
    buckets = backend.saver.prepare_write_data(cid, items, resolver, "data", bucket_count=bucket_count)
    results = backend.saver.write_data(cid, buckets, replicate_after_write=replicate,
                                       thread_count=bucket_count if thread_count is None else thread_count)
    return buckets, sorted(results, key=lambda r: r.index.fqn)


# ---- the record format (test_checkpoint_saver.py:145-187, :905-960) ----------------------------------------------------
REFERENCE_TENSORS = [
    torch.tensor([1, 2, 3], dtype=torch.int32),
    torch.tensor([[1, 2], [3, 4]], dtype=torch.float32),
    torch.tensor([[[1], [2]], [[3], [4]]], dtype=torch.float16),
    torch.tensor([1, 2, 3], dtype=torch.int64),
    torch.tensor([1.5, 2.5], dtype=torch.bfloat16),
    torch.tensor([[1.0, 2.0, 3.0]], dtype=torch.float32),
    torch.tensor([], dtype=torch.float32),
    torch.tensor([[[]]], dtype=torch.int32),
]


@pytest.mark.parametrize("case", range(len(REFERENCE_TENSORS)))
def test_record_is_length_prefixed_header_then_raw_bytes(backend, tmp_path, case):
    tensor = REFERENCE_TENSORS[case]
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_optimized"))
    buckets, results = _save(backend, cid, {"test_tensor": tensor})
    assert len(results) == 1 and results[0].storage_data.offset == 0
    path = os.path.join(cid.data, buckets[0].object_name)
    raw = open(path, "rb").read()
    assert raw[8:16] == b"MLF_TENS"
    assert struct.unpack("<Q", raw[:8])[0] == len(raw) - METADATA_SIZE == results[0].storage_data.length
    assert raw[16:METADATA_SIZE] == bytes(METADATA_SIZE - 16)
    (header_len,) = struct.unpack("<I", raw[METADATA_SIZE : METADATA_SIZE + 4])
    assert results[0].size_in_bytes == 4 + header_len + tensor.numel() * tensor.element_size()  # empty: header only
    _assert_tensor_record(path, 0, results[0].storage_data.length, tensor)


# ---- prepare_write_data (:858-1050) -------------------------------------------------------------------------------------
def test_prepare_single_items_and_names(backend, tmp_path):
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_prepare_single"))
    tensor = torch.tensor([1, 2, 3])
    items, resolver = _plan(backend, {"item_0": tensor})
    buckets = backend.saver.prepare_write_data(cid, items, resolver, object_name_prefix="data", bucket_count=1)
    assert len(buckets) == 1 and buckets[0].object_name == "data_0_src0.distcp"
    assert buckets[0].object_id == CheckpointObjectId.from_container(cid, "data_0_src0.distcp")
    assert len(buckets[0].tensor_data) == 1 and len(buckets[0].bytesio_data) == 0
    assert buckets[0].tensor_data[0][0] is items[0]
    if backend.name == "oracle":                            # the gfx950 saver hands on a placeholder for the packed image
        assert torch.equal(buckets[0].tensor_data[0][1], tensor)
    items, resolver = _plan(backend, {"item_0": b"test byte data"})
    buckets = backend.saver.prepare_write_data(cid, items, resolver, object_name_prefix="data", bucket_count=1)
    assert len(buckets) == 1 and buckets[0].object_name == "data_0_src0.distcp"
    assert len(buckets[0].bytesio_data) == 1 and len(buckets[0].tensor_data) == 0
    assert buckets[0].bytesio_data[0][1].getvalue() == b"test byte data"


@pytest.mark.parametrize("bucket_count", [1, 2, 3])
def test_prepare_distributes_every_item_once(backend, tmp_path, bucket_count):
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_prepare_mixed"))
    entries = {"item_0_tensor": torch.tensor([1, 2, 3]), "item_1_bytes": b"test byte data",
               "item_2_tensor": torch.tensor([7, 8, 9])}
    items, resolver = _plan(backend, entries)
    buckets = backend.saver.prepare_write_data(cid, items, resolver, object_name_prefix="data", bucket_count=bucket_count)
    assert 0 < len(buckets) <= bucket_count
    assert [b.object_name for b in buckets] == [f"data_{k}_src0.distcp" for k in range(len(buckets))]
    tensor_fqns = sorted(i.index.fqn for b in buckets for i, _ in b.tensor_data)
    blob_values = [d.getvalue() for b in buckets for _, d in b.bytesio_data]
    assert tensor_fqns == ["item_0_tensor", "item_2_tensor"] and blob_values == [b"test byte data"]
    two = {"item_0": torch.tensor([1, 2, 3]), "item_1": torch.tensor([4, 5, 6])}
    items, resolver = _plan(backend, two)
    buckets = backend.saver.prepare_write_data(cid, items, resolver, object_name_prefix="data", bucket_count=min(bucket_count, 2))
    assert len(buckets) == min(bucket_count, 2)             # two equal tensors spread over two buckets
    assert sorted(i.index.fqn for b in buckets for i, _ in b.tensor_data) == ["item_0", "item_1"]


def test_prepare_nothing_and_resolver_failure(backend, tmp_path):
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_prepare_empty"))
    assert backend.saver.prepare_write_data(cid, [], _Resolver({}), object_name_prefix="data", bucket_count=1) == []
    with pytest.raises(KeyError):
        backend.saver.prepare_write_data(cid, [_tensor_item("item_0", torch.tensor([1, 2, 3]))], _Resolver({}),
                                         object_name_prefix="data", bucket_count=1)


def test_prepare_copies_host_views_only(tmp_path):
    """Host tensors that are views or non-contiguous are copied so that training may go on writing the parent;
    whole contiguous tensors and tensors on a device are handed on untouched (:1052-1140)."""
    saver = OracleCheckpointSaver()
    contig, non_contig, view = torch.randn(10), torch.randn(10, 2).t(), torch.randn(20)[2:5]
    on_device = torch.empty(4, 3, device="meta").t()        # not on the host: must come through as it is
    entries = {"contig": contig, "non_contig": non_contig, "view": view, "device": on_device}
    items = [_tensor_item(k, v) for k, v in entries.items()]
    resolver = _Resolver({MetadataIndex(fqn=k): v for k, v in entries.items()})
    bucket = saver.prepare_write_data(CheckpointContainerId(str(tmp_path / "c")), items, resolver, "data", 1)[0]
    got = {item.index.fqn: t for item, t in bucket.tensor_data}
    assert got["contig"].is_contiguous() and got["contig"].data_ptr() == contig.data_ptr()
    assert got["non_contig"].is_contiguous() and got["non_contig"].data_ptr() != non_contig.data_ptr()
    assert torch.equal(got["non_contig"], non_contig)
    assert got["view"].is_contiguous() and got["view"].data_ptr() != view.data_ptr() and torch.equal(got["view"], view)
    assert got["view"].untyped_storage().size() == got["view"].numel() * got["view"].itemsize
    assert got["device"].device.type == "meta" and not got["device"].is_contiguous()


# ---- write_data (:1151-1600) ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("thread_count", [1, 2, 3])
def test_write_single_tensor_and_single_blob(backend, tmp_path, thread_count):
    cid = CheckpointContainerId(str(tmp_path / f"checkpoint_write_data_th{thread_count}"))
    tensor = torch.tensor([1, 2, 3])
    buckets, results = _save(backend, cid, {"item_0": tensor}, bucket_count=thread_count)
    assert len(results) == 1 and results[0].index == MetadataIndex(fqn="item_0")
    info = results[0].storage_data
    assert (info.relative_path, info.offset) == ("data_0_src0.distcp", 0) and results[0].size_in_bytes == info.length > 0
    _assert_tensor_record(os.path.join(cid.data, info.relative_path), 0, info.length, tensor)
    cid = CheckpointContainerId(str(tmp_path / f"checkpoint_write_data_bytes_th{thread_count}"))
    buckets, results = _save(backend, cid, {"item_0": b"test byte data"}, bucket_count=thread_count)
    info = results[0].storage_data
    assert (info.relative_path, info.offset, info.length) == ("data_0_src0.distcp", 0, 14)
    assert results[0].size_in_bytes == 14
    raw = open(os.path.join(cid.data, info.relative_path), "rb").read()
    assert raw[METADATA_SIZE:] == b"test byte data" and len(raw) == METADATA_SIZE + 14


@pytest.mark.parametrize("thread_count", [1, 2, 3])
def test_write_mixed_items_offsets_are_sequential_per_object(backend, tmp_path, thread_count):
    cid = CheckpointContainerId(str(tmp_path / f"checkpoint_write_data_mixed_th{thread_count}"))
    entries = {"item_0_tensor": torch.tensor([1, 2, 3]), "item_1_bytes": b"test byte data",
               "item_2_tensor": torch.tensor([7, 8, 9])}
    buckets, results = _save(backend, cid, entries, bucket_count=thread_count)
    assert [r.index.fqn for r in results] == list(entries)
    where = {i.index.fqn: b.object_name for b in buckets for i, _ in list(b.tensor_data) + list(b.bytesio_data)}
    assert all(r.storage_data.relative_path == where[r.index.fqn] for r in results)
    assert results[0].size_in_bytes > 0 and results[1].size_in_bytes == 14 and results[2].size_in_bytes > 0
    by_file = {}
    for r in results:
        by_file.setdefault(r.storage_data.relative_path, []).append(r)
    for name, group in by_file.items():
        path = os.path.join(cid.data, name)
        expected_offset = 0
        kinds = []
        for r in sorted(group, key=lambda r: r.storage_data.offset):
            assert r.storage_data.offset == expected_offset   # no gaps, no padding
            value = entries[r.index.fqn]
            if isinstance(value, bytes):
                with open(path, "rb") as f:
                    f.seek(METADATA_SIZE + r.storage_data.offset)
                    assert f.read(r.storage_data.length) == value
            else:
                _assert_tensor_record(path, r.storage_data.offset, r.storage_data.length, value)
            kinds.append(isinstance(value, bytes))
            expected_offset += r.storage_data.length
        assert kinds == sorted(kinds)                          # tensors first, byte items behind them
        assert os.path.getsize(path) == METADATA_SIZE + expected_offset


@pytest.mark.parametrize("thread_count", [1, 2, 3])
def test_write_multiple_tensors(backend, tmp_path, thread_count):
    cid = CheckpointContainerId(str(tmp_path / f"checkpoint_write_data_multi_th{thread_count}"))
    entries = {"item_0": torch.tensor([1, 2, 3]), "item_1": torch.tensor([4, 5, 6])}
    buckets, results = _save(backend, cid, entries, bucket_count=thread_count)
    assert len(results) == 2
    if thread_count == 1:
        assert results[0].storage_data.offset == 0 and results[1].storage_data.offset == results[0].size_in_bytes
        assert {r.storage_data.relative_path for r in results} == {"data_0_src0.distcp"}
    else:
        assert sorted(r.storage_data.relative_path for r in results) == ["data_0_src0.distcp", "data_1_src0.distcp"]
        assert all(r.storage_data.offset == 0 for r in results)
    for r in results:
        _assert_tensor_record(os.path.join(cid.data, r.storage_data.relative_path), r.storage_data.offset,
                              r.storage_data.length, entries[r.index.fqn])


def test_write_ten_items_over_four_buckets(backend, tmp_path):
    cid = CheckpointContainerId(str(tmp_path / "ckpt_threads_multi"))
    entries = {f"item_{i}": torch.tensor([i], dtype=torch.int32) for i in range(10)}
    buckets, results = _save(backend, cid, entries, bucket_count=4)
    assert len(buckets) == 4 and len(results) == 10
    for r in results:
        _assert_tensor_record(os.path.join(cid.data, r.storage_data.relative_path), r.storage_data.offset,
                              r.storage_data.length, entries[r.index.fqn])


@pytest.mark.parametrize("thread_count", [1, 2, 3])
def test_write_no_buckets_creates_nothing(backend, tmp_path, thread_count):
    cid = CheckpointContainerId(str(tmp_path / f"checkpoint_write_data_empty_th{thread_count}"))
    os.makedirs(cid.data)
    assert backend.saver.write_data(cid, write_buckets=[], thread_count=thread_count, replicate_after_write=False) == []
    assert not os.listdir(cid.data)


@pytest.mark.parametrize("preexisting_content", [b"", b"some old data"])
def test_write_replaces_a_file_that_is_in_the_way(backend, tmp_path, preexisting_content):
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_write_data_overwrite"))
    os.makedirs(cid.data)
    tensor = torch.tensor([1, 2, 3])
    items, resolver = _plan(backend, {"item_0": tensor})
    buckets = backend.saver.prepare_write_data(cid, items, resolver, "data", bucket_count=1)
    path = os.path.join(cid.data, buckets[0].object_name)
    with open(path, "wb") as f:
        f.write(preexisting_content)
    results = backend.saver.write_data(cid, buckets, thread_count=1, replicate_after_write=False)
    assert len(results) == 1 and results[0].storage_data.relative_path == buckets[0].object_name
    _assert_tensor_record(path, 0, results[0].storage_data.length, tensor)
    assert os.path.getsize(path) == METADATA_SIZE + results[0].storage_data.length


@pytest.mark.parametrize("thread_count", [0, -1, -5])
def test_write_thread_count_below_one_is_one(backend, tmp_path, thread_count):
    cid = CheckpointContainerId(str(tmp_path / f"checkpoint_write_data_tensor_th{thread_count}"))
    entries = {"item_0": torch.tensor([1, 2, 3]), "item_1": torch.tensor([4, 5, 6])}
    buckets, results = _save(backend, cid, entries, bucket_count=1, thread_count=thread_count)
    assert [r.storage_data.relative_path for r in results] == ["data_0_src0.distcp"] * 2
    assert results[0].storage_data.offset == 0 and results[1].storage_data.offset == results[0].size_in_bytes
    for r in results:
        _assert_tensor_record(os.path.join(cid.data, "data_0_src0.distcp"), r.storage_data.offset,
                              r.storage_data.length, entries[r.index.fqn])


def test_oracle_write_restores_the_torch_thread_count(tmp_path):
    """The intra-op thread count the reference lowers while writing is put back, also when there is nothing to
    write (:240-272); the rule for the lowered value is cpus // 2 // ranks // threads, at least 1 (:443-450)."""
    saver = OracleCheckpointSaver(accelerator_count=2)
    before = torch.get_num_threads()
    saver.write_data(CheckpointContainerId(str(tmp_path / "ckpt_threads")), [], replicate_after_write=False, thread_count=1)
    assert torch.get_num_threads() == before
    cpus = os.cpu_count() or 1
    assert saver.torch_thread_count(1) == max(1, cpus // 2 // 2) and saver.torch_thread_count(4) == max(1, cpus // 2 // 2 // 4)
    assert OracleCheckpointSaver(accelerator_count=0).torch_thread_count(0) == max(1, cpus // 2)


@GPU
@pytest.mark.parametrize("thread_count", [1, 2, 3])
def test_hip_write_reports_a_failing_buffer(tmp_path, thread_count, monkeypatch):
    backend = _Backend("hip")
    cid = CheckpointContainerId(str(tmp_path / f"checkpoint_write_data_io_error_th{thread_count}"))
    items, resolver = _plan(backend, {"item_0": torch.tensor([1, 2, 3])})
    buckets = backend.saver.prepare_write_data(cid, items, resolver, "data", bucket_count=thread_count)

    def failing(*args, **kwargs):
        raise IOError("Test IOError")

    monkeypatch.setattr(backend.saver._chkpt_obj_manager, "acquire_buffer", failing)
    with pytest.raises(IOError, match="Test IOError"):
        backend.saver.write_data(cid, buckets, thread_count=thread_count, replicate_after_write=False)


@GPU
def test_hip_write_hands_the_object_to_replication_only_when_asked(tmp_path):
    backend = _Backend("hip")
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_write_data_no_replication"))
    _save(backend, cid, {"item_0": torch.tensor([1, 2, 3])}, replicate=False)
    assert backend.replication.calls == []
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_write_data_replication"))
    buckets, _ = _save(backend, cid, {"item_0": torch.tensor([1, 2, 3])}, replicate=True)
    assert len(backend.replication.calls) == 1
    handed = backend.replication.calls[0]
    assert isinstance(handed, BufferIO) and handed.is_readonly
    assert handed.buffer_obj.get_id() == str(CheckpointObjectId.from_container(cid, buckets[0].object_name))
    handed.close()


# ---- write_metadata / read_metadata (saver :1760-1867, loader :160-203): host logic, no GPU needed ------------------------
def _host_saver(kind):
    if kind == "oracle":
        return OracleCheckpointSaver()
    from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver

    return HipMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, CheckpointObjectManager(), None)


def _host_loader(kind):
    if kind == "oracle":
        return OracleCheckpointLoader()
    from ml_flashpoint.hip.checkpoint_loader import HipMLFlashpointCheckpointLoader

    return HipMLFlashpointCheckpointLoader(CheckpointObjectManager(), None)


def _reference_metadata():
    return torchdistmeta.Metadata(
        state_dict_metadata={
            "model.layer1.weight": torchdistmeta.TensorStorageMetadata(
                properties=torchdistmeta.TensorProperties(dtype=torch.float32, layout=torch.strided),
                size=torch.Size([10, 20]), chunks=[]),
            "model.layer2.bias": torchdistmeta.TensorStorageMetadata(
                properties=torchdistmeta.TensorProperties(dtype=torch.float16, layout=torch.strided),
                size=torch.Size([30]), chunks=[]),
            "some_bytes": torchdistmeta.BytesStorageMetadata(),
        },
        storage_data={
            "model.layer1.weight": {"relative_path": "data_0_src0.distcp", "offset": 0, "length": 800},
            "model.layer2.bias": {"relative_path": "data_1_src0.distcp", "offset": 100, "length": 60},
            "some_bytes": {"relative_path": "data_1_src0.distcp", "offset": 160, "length": 20},
        },
    )


@pytest.mark.parametrize("kind", ["oracle", "hip"])
def test_metadata_is_written_through_a_temporary_file(kind, tmp_path, monkeypatch):
    saver, loader, metadata = _host_saver(kind), _host_loader(kind), _reference_metadata()
    cid = CheckpointContainerId(str(tmp_path / "checkpoint_1"))          # not created yet: the call makes it
    saver.write_metadata(cid, metadata)
    path = os.path.join(cid.data, ".metadata")
    assert pickle.load(open(path, "rb")) == metadata and not os.path.exists(path + ".tmp")
    assert loader.read_metadata(cid) == metadata
    saver.write_metadata(cid, metadata, md_object_name="custom.meta")
    assert pickle.load(open(os.path.join(cid.data, "custom.meta"), "rb")) == metadata
    assert not os.path.exists(os.path.join(cid.data, "custom.meta.tmp"))
    assert loader.read_metadata(cid, object_name="custom.meta") == metadata
    with pytest.raises(FileNotFoundError):
        loader.read_metadata(cid, object_name="non_existent.pt")
    with open(os.path.join(cid.data, "invalid_metadata.pt"), "w") as f:
        f.write("this is not a valid metadata file")
    with pytest.raises(Exception):
        loader.read_metadata(cid, object_name="invalid_metadata.pt")

    blocked = CheckpointContainerId(str(tmp_path / "checkpoint_3"))
    os.makedirs(os.path.join(blocked.data, ".metadata"))                  # a directory where the file should go
    with pytest.raises(OSError):
        saver.write_metadata(blocked, metadata)
    assert os.path.exists(os.path.join(blocked.data, ".metadata.tmp"))    # kept, to be looked at

    failing = CheckpointContainerId(str(tmp_path / "checkpoint_write_fail"))

    def broken_dump(*args, **kwargs):
        raise Exception("Simulated write error")

    monkeypatch.setattr(pickle, "dump", broken_dump)
    with pytest.raises(Exception, match="Simulated write error"):
        saver.write_metadata(failing, metadata)
    assert os.path.exists(os.path.join(failing.data, ".metadata.tmp"))
    assert not os.path.exists(os.path.join(failing.data, ".metadata"))    # the rename was never reached


# ---- read_data (loader :223-380, :542-728) ----------------------------------------------------------------------------------
def _read_item(kind, storage_index, offsets, lengths, fqn="dest"):
    return ReadItem(type=kind, storage_index=storage_index, storage_offsets=torch.Size(offsets),
                    lengths=torch.Size(lengths), dest_index=MetadataIndex(fqn=fqn), dest_offsets=torch.Size([0] * len(offsets)))


class _Planner:
    def __init__(self, target=None):
        self.target, self.resolved, self.committed, self.loaded = target, [], [], []

    def resolve_tensor(self, req):
        self.resolved.append(req)
        return self.target

    def commit_tensor(self, req, tensor):
        self.committed.append((req, tensor))

    def load_bytes(self, req, value):
        self.loaded.append((req, value.read()))


@pytest.fixture
def two_item_object(backend, tmp_path):
    """The object the reference's loader tests read: a 4x5 int32 ``arange`` and a pickled dict behind it."""
    cid = CheckpointContainerId(str(tmp_path / "ckpt"))
    blob = pickle.dumps({"key": "value", "count": 100})
    buckets, results = _save(backend, cid, {"a_tensor": torch.arange(20, dtype=torch.int32).reshape(4, 5), "b_bytes": blob})
    storage = {i: _StorageInfo(r.storage_data.relative_path, r.storage_data.offset, r.storage_data.length)
               for i, r in enumerate(results)}
    return CheckpointObjectId.from_container(cid, buckets[0].object_name), storage


def test_read_a_tensor_slice(backend, two_item_object):
    oid, storage = two_item_object
    target = torch.empty(2, 3, dtype=torch.int32, device=backend.device)
    req = _read_item(LoadItemType.TENSOR, 0, (1, 1), (2, 3))
    planner = _Planner(target)
    backend.loader.read_data(oid, [req], planner, storage)
    expected = torch.tensor([[6, 7, 8], [11, 12, 13]], dtype=torch.int32)
    assert planner.resolved == [req] and len(planner.committed) == 1 and planner.committed[0][0] == req
    assert torch.equal(planner.committed[0][1].cpu(), expected) and torch.equal(target.cpu(), expected)
    assert planner.loaded == []


def test_read_bytes_and_mixed_requests(backend, two_item_object):
    oid, storage = two_item_object
    req_bytes = _read_item(LoadItemType.BYTE_IO, 1, (0, 0), (0, 0))
    planner = _Planner()
    backend.loader.read_data(oid, [req_bytes], planner, storage)
    assert planner.resolved == [] and planner.committed == [] and len(planner.loaded) == 1
    assert planner.loaded[0][0] == req_bytes and pickle.loads(planner.loaded[0][1]) == {"key": "value", "count": 100}
    target = torch.empty(4, 5, dtype=torch.int32, device=backend.device)
    req_tensor = _read_item(LoadItemType.TENSOR, 0, (0, 0), (4, 5))
    planner = _Planner(target)
    backend.loader.read_data(oid, [req_tensor, req_bytes], planner, storage)
    assert planner.resolved == [req_tensor] and planner.committed[0][0] == req_tensor
    assert torch.equal(planner.committed[0][1].cpu(), torch.arange(20, dtype=torch.int32).reshape(4, 5))
    assert pickle.loads(planner.loaded[0][1]) == {"key": "value", "count": 100}


def test_read_into_a_target_of_the_wrong_size(backend, two_item_object):
    oid, storage = two_item_object
    planner = _Planner(torch.empty(5, 5, dtype=torch.int32, device=backend.device))
    with pytest.raises(AssertionError, match="mismatch sizes"):
        backend.loader.read_data(oid, [_read_item(LoadItemType.TENSOR, 0, (1, 1), (2, 3))], planner, storage)
    assert planner.committed == []


@pytest.mark.parametrize(
    "stored, offsets, lengths, expected",
    [
        (torch.arange(20, dtype=torch.float32), (5,), (10,), torch.arange(5, 15, dtype=torch.float32)),
        (torch.arange(20, dtype=torch.int64).reshape(4, 5), (1, 2), (2, 3), torch.tensor([[7, 8, 9], [12, 13, 14]])),
        (torch.arange(60, dtype=torch.float32).reshape(3, 4, 5), (1, 1, 2), (2, 2, 3),
         torch.arange(60, dtype=torch.float32).reshape(3, 4, 5)[1:3, 1:3, 2:5]),
    ],
    ids=["1d", "2d", "3d"],
)
def test_read_known_sub_boxes(backend, tmp_path, stored, offsets, lengths, expected):
    cid = CheckpointContainerId(str(tmp_path / "ckpt"))
    buckets, results = _save(backend, cid, {"t": stored})
    storage = {0: _StorageInfo(results[0].storage_data.relative_path, 0, results[0].storage_data.length)}
    target = torch.zeros(lengths, dtype=stored.dtype, device=backend.device)
    backend.loader.read_data(CheckpointObjectId.from_container(cid, buckets[0].object_name),
                             [_read_item(LoadItemType.TENSOR, 0, offsets, lengths)], _Planner(target), storage)
    assert torch.equal(target.cpu(), expected)


def test_read_a_missing_object(backend, tmp_path):
    with pytest.raises(FileNotFoundError, match="does not exist on any node in the cluster"):
        backend.loader.read_data(CheckpointObjectId(str(tmp_path / "ckpt" / "gone.distcp")),
                                 [_read_item(LoadItemType.TENSOR, 0, (0,), (1,))], _Planner(torch.zeros(1)), {})


# ---- read_tensor on the host (loader :223-380) ---------------------------------------------------------------------------------
def _torch_saved(tensor):
    stream = io.BytesIO()
    torch.save(tensor, stream)
    stream.seek(0)
    return stream


@pytest.mark.parametrize(
    "stored, offsets, lengths, expected",
    [
        (torch.arange(20, dtype=torch.float32), (5,), (10,), torch.arange(5, 15, dtype=torch.float32)),
        (torch.arange(20, dtype=torch.int64).reshape(4, 5), (1, 2), (2, 3),
         torch.tensor([[7, 8, 9], [12, 13, 14]], dtype=torch.int64)),
        (torch.arange(60, dtype=torch.float32).reshape(3, 4, 5), (1, 0, 3), (2, 2, 2),
         torch.tensor([[[23.0, 24.0], [28.0, 29.0]], [[43.0, 44.0], [48.0, 49.0]]])),
    ],
    ids=["1d", "2d", "3d"],
)
@pytest.mark.parametrize("optimized", [False, True], ids=["legacy-loader", "optimized-loader"])
def test_read_tensor_known_slices_of_a_torch_saved_record(stored, offsets, lengths, expected, optimized):
    """A ``torch.save`` record is read by either loader setting: its first four bytes give a length far above the
    limit for a header, so the optimized loader falls back (loader tests :223-302, :359-380)."""
    got = _host_loader("hip").read_tensor(_torch_saved(stored), _read_item(LoadItemType.TENSOR, 0, offsets, lengths),
                                     use_optimized_loader=optimized)
    assert got.dtype == expected.dtype and torch.equal(got, expected)


def test_read_tensor_of_a_header_record():
    """Length, pickled header, raw bytes (loader test :322-357); the stream may start anywhere."""
    tensor = torch.tensor([1, 2, 3], dtype=torch.int32)
    stream = io.BytesIO()
    stream.write(b"skipped")
    stream.write(TensorHeader(dtype=tensor.dtype, shape=tensor.shape).to_bytes())
    stream.write(tensor.numpy().tobytes())
    stream.seek(len(b"skipped"))
    got = _host_loader("hip").read_tensor(stream, _read_item(LoadItemType.TENSOR, 0, (0,), (3,)), use_optimized_loader=True)
    assert got.dtype == torch.int32 and torch.equal(got, tensor)
    stream.seek(len(b"skipped"))
    with pytest.raises(Exception):  # without the optimized loader the record is handed to torch.load, which rejects it
        _host_loader("hip").read_tensor(stream, _read_item(LoadItemType.TENSOR, 0, (0,), (3,)))


def test_read_tensor_of_bytes_that_are_no_record():
    with pytest.raises(IndexError):  # what torch.load raises for this text (loader test :304-320)
        _host_loader("hip").read_tensor(io.BytesIO(b"this is not a valid tensor"), _read_item(LoadItemType.TENSOR, 0, (0,), (1,)))
    header = TensorHeader(dtype=torch.float32, shape=torch.Size([4])).to_bytes()
    with pytest.raises(Exception):  # a header whose payload is cut short
        _host_loader("hip").read_tensor(io.BytesIO(header + b"\0" * 15), _read_item(LoadItemType.TENSOR, 0, (0,), (4,)),
                                   use_optimized_loader=True)
