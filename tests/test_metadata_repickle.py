"""The metadata object's bytes from one save to the next (``repickled_with_storage_meta``), CPU only.

A run that keeps its DCP plan writes, save after save, a metadata object that differs in ``storage_meta`` only (the
checkpoint's path and the save's id).  The writer then takes the previous bytes and exchanges that part instead of
pickling tens of thousands of entries again.  The bar here: the result is byte for byte what ``pickle.dumps`` makes
of the new object - for paths of any length and alphabet, objects of one frame and of many - and wherever the
short cut cannot be taken safely the function says so (None) instead of returning bytes.
"""

import concurrent.futures
import dataclasses
import os
import pickle

import pytest
import torch
import torch.multiprocessing as torch_mp
from hypothesis import given, settings
from hypothesis import strategies as st
from torch.distributed.checkpoint import DefaultSavePlanner
from torch.distributed.checkpoint.filesystem import _StorageInfo
from torch.distributed.checkpoint.metadata import Metadata, MetadataIndex, StorageMeta
from torch.distributed.checkpoint.utils import _DistWrapper

from ml_flashpoint.adapter.pytorch import custom_state_dict_saver as three_calls
from ml_flashpoint.adapter.pytorch import memory_storage_writer as msw
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter, repickled_with_storage_meta
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
from oracle.cpu_path import OracleCheckpointSaver

pytestmark = pytest.mark.filterwarnings("ignore:torch.distributed is disabled")


def _metadata(n_tensors: int) -> Metadata:
    """A metadata object as DCP's planner makes it, with ``storage_data`` filled the way ``finish_checkpoint`` does."""
    sd = {f"layer.{i}.weight": torch.zeros(3, i % 5 + 1, dtype=(torch.float32, torch.bfloat16, torch.int64)[i % 3])
          for i in range(n_tensors)}
    sd["extra.step"] = 17  # a non-tensor entry
    planner = DefaultSavePlanner()
    planner.set_up_planner(sd, is_coordinator=True)
    _, md = planner.create_global_plan([planner.create_local_plan()])
    where, offset = {}, 0
    for fqn, entry in md.state_dict_metadata.items():
        index = MetadataIndex(fqn, entry.chunks[0].offsets if hasattr(entry, "chunks") else None)
        where[index] = _StorageInfo(relative_path="__0__0_src0.distcp", offset=offset, length=100 + len(fqn))
        offset += 100 + len(fqn)
    return dataclasses.replace(md, storage_data=where)


def _meta(path: str, save_id: str = "7a9b-opulent-otter") -> StorageMeta:
    return StorageMeta(checkpoint_id=path, save_id=save_id)


@pytest.mark.parametrize("n_tensors", [0, 3, 400, 6000])
@pytest.mark.parametrize("old_path, new_path", [
    ("/dev/shm/run/step-100_ckpt", "/dev/shm/run/step-200_ckpt"),          # same length
    ("/dev/shm/run/step-99_ckpt", "/dev/shm/run/step-100_ckpt"),           # one byte longer
    ("/dev/shm/run/step-1000_ckpt", "/dev/shm/run/step-7_ckpt"),           # shorter
    ("/tmp/" + "d" * 240 + "/step-9_ckpt", "/tmp/" + "d" * 240 + "/step-10_ckpt"),  # across the 255-byte string form
    ("/tmp/ckpt/шаг-1", "/tmp/ckpt/步-22"),                                  # not ASCII
])
def test_exchanged_storage_meta_gives_the_bytes_of_a_fresh_pickle(n_tensors, old_path, new_path):
    md = _metadata(n_tensors)
    old, new = _meta(old_path, "save-one"), _meta(new_path, "save-number-two")
    before = pickle.dumps(dataclasses.replace(md, storage_meta=old))
    got = repickled_with_storage_meta(before, md, old, new)
    fresh = dataclasses.replace(md, storage_meta=new)
    assert got is not None
    assert got == pickle.dumps(fresh)
    assert pickle.loads(got) == fresh
    if n_tensors >= 6000:
        assert before.count(b"\x95") > 3 and len(before) > 3 * 65536  # several frames: only the last one changes


@settings(max_examples=60, deadline=None)
@given(st.text(min_size=0, max_size=600), st.text(min_size=0, max_size=600), st.text(max_size=40), st.text(max_size=40))
def test_any_path_and_save_id(old_path, new_path, old_id, new_id):
    md = _metadata(40)
    old, new = _meta(old_path, old_id), _meta(new_path, new_id)
    before = pickle.dumps(dataclasses.replace(md, storage_meta=old))
    got = repickled_with_storage_meta(before, md, old, new)
    fresh = dataclasses.replace(md, storage_meta=new)
    # Where the function answers, its answer loads as the new object; it declines where the part to be exchanged
    # refers to an object by memo number (the same string object twice: '' and one-character strings are singletons)
    if got is not None:
        assert pickle.loads(got) == fresh
    distinct = len({id(x) for x in (old_path, old_id)}) == 2 and len({id(x) for x in (new_path, new_id)}) == 2
    if distinct and min(len(x) for x in (old_path, old_id, new_path, new_id)) > 1:
        assert got == pickle.dumps(fresh)


def test_the_same_string_object_twice_in_the_new_part_is_declined():
    """'' is one object in CPython: as path and as save id it is pickled once and referred to by memo number the
    second time - a number that is another one in the stand-in than in the real object."""
    md = _metadata(40)
    old, new = _meta("0", ""), _meta("", "")
    before = pickle.dumps(dataclasses.replace(md, storage_meta=old))
    got = repickled_with_storage_meta(before, md, old, new)
    assert got is None or pickle.loads(got) == dataclasses.replace(md, storage_meta=new)
    twice = "/run/step-3_ckpt"
    new2 = _meta(twice, twice)
    got = repickled_with_storage_meta(before, md, old, new2)
    assert got is None


def test_declines_when_the_old_bytes_are_not_what_they_are_said_to_be():
    md = _metadata(50)
    old, new = _meta("/a/step-1_ckpt"), _meta("/a/step-2_ckpt")
    before = pickle.dumps(dataclasses.replace(md, storage_meta=old))
    assert repickled_with_storage_meta(before, md, _meta("/a/step-3_ckpt"), new) is None  # another storage_meta inside
    assert repickled_with_storage_meta(before, md, None, new) is None
    assert repickled_with_storage_meta(before[:-1], md, old, new) is None                   # truncated
    assert repickled_with_storage_meta(b"", md, old, new) is None
    assert repickled_with_storage_meta(pickle.dumps(dataclasses.replace(md, storage_meta=old), protocol=3), md, old, new) is None
    # an object whose tail is spread over two frames is left alone: a storage_meta of more than one frame's size
    huge = _meta("/x" * 70000)
    assert repickled_with_storage_meta(pickle.dumps(dataclasses.replace(md, storage_meta=huge)), md, huge, new) is None
    # a path that occurs earlier in the object as the same string object is a back-reference in the real pickle
    shared = "/a/step-5_ckpt"
    md2 = dataclasses.replace(md, planner_data={"note": shared})
    old2 = _meta(shared)
    got = repickled_with_storage_meta(pickle.dumps(dataclasses.replace(md2, storage_meta=old2)), md2, old2, new)
    assert got is None or pickle.loads(got) == dataclasses.replace(md2, storage_meta=new)


# ---- through the writer: three saves of a kept plan ------------------------------------------------------------------


@pytest.fixture(scope="module")
def manager_future():
    mgr = torch_mp.get_context("spawn").Manager()
    fut = concurrent.futures.Future()
    fut.set_result(mgr)
    yield fut
    mgr.shutdown()


class _PredictingSaver(OracleCheckpointSaver):
    """The oracle's saver with the three optional members the writer looks for.  It predicts what the last write of
    the same items returned (the gfx950 saver predicts from its layout); ``same_objects`` says whether a write then
    returns those very objects or equal ones."""

    def __init__(self, same_objects: bool, **kw):
        super().__init__(**kw)
        self.same_objects = same_objects
        self.last_write_locations = None
        self.last_global_metadata = None
        self.last_metadata_pickle = None
        self.wrote = []  # "bytes" / "object" per metadata object written
        self._seen = None  # (items, results) of the last write

    def _items(self, buckets):
        return [item for b in buckets for item, _ in list(b.tensor_data) + list(b.bytesio_data)]

    def predict_write_results(self, buckets):
        items = self._items(buckets)
        if self._seen is None or len(items) != len(self._seen[0]) or any(a is not b for a, b in zip(items, self._seen[0])):
            return None
        return list(self._seen[1])

    def write_data(self, checkpoint_id, write_buckets, replicate_after_write, thread_count=1):
        results = super().write_data(checkpoint_id, write_buckets, replicate_after_write, thread_count)
        by_index = {r.index: r for r in results}
        ordered = [by_index[item.index] for item in self._items(write_buckets)]
        if self._seen is not None and self.same_objects and [r.index for r in self._seen[1]] == [r.index for r in ordered] \
                and all(a == b for a, b in zip(self._seen[1], ordered)):
            ordered = self._seen[1]
        self._seen = (self._items(write_buckets), ordered)
        return list(ordered)

    def write_metadata(self, checkpoint_id, metadata, md_object_name=".metadata"):
        self.wrote.append("object")
        return super().write_metadata(checkpoint_id, metadata, md_object_name)

    def write_metadata_bytes(self, checkpoint_id, pickled, md_object_name=".metadata"):
        self.wrote.append("bytes")
        path = os.path.join(checkpoint_id.data, md_object_name)
        with open(path, "wb") as f:
            f.write(pickled)


@pytest.mark.parametrize("same_objects", [True, False])
def test_saves_of_a_kept_plan_reuse_the_previous_bytes(shm_dir, manager_future, same_objects, monkeypatch):
    saver = _PredictingSaver(same_objects)
    dist = _DistWrapper(None, False, 0)
    sd = {f"w{i}": torch.full((4, 3), float(i)) for i in range(30)}
    sd["step"] = 5
    cached, metadata = None, None
    respliced, payloads = [], []
    made = msw._EarlyMetadata.result_for

    def watched(self, *a, **k):
        out = made(self, *a, **k)
        respliced.append(self.respliced)
        return out

    monkeypatch.setattr(msw._EarlyMetadata, "result_for", watched)
    for step in range(1, 7):
        cid = CheckpointContainerId(os.path.join(shm_dir, f"step-{step}_ckpt"))
        saver.initialize_checkpoint(cid)
        writer = MemoryStorageWriter(saver, manager_future)
        writer.reset(cid.data)
        if step == 5:
            sd["w3"] = torch.full((9, 3), 3.0)  # another shape: another plan, other offsets
            cached = None
        buckets, md, central, local, validated = three_calls.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist, cached)
        metadata = md if md is not None else metadata
        cached = (central, local, validated)
        if md is None:
            writer.expect_metadata(metadata)
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets)
        three_calls.write_data(cid, writer, staged, replicate_after_write=False)
        three_calls.finish_write(cid, writer, metadata, dist)
        saver.finalize_checkpoint(cid)
        raw = open(os.path.join(cid.data, ".metadata"), "rb").read()
        payloads.append(raw)
        got = pickle.loads(raw)
        assert got.storage_meta.checkpoint_id == cid.data and got.storage_meta.save_id == writer._current_save_id
        assert got.state_dict_metadata == metadata.state_dict_metadata and got.storage_data == metadata.storage_data
        assert got == metadata  # (finish_checkpoint has put storage_data and storage_meta into the caller's object)
    # save 1 and 2 build and validate the plan (items differ: nothing predicted), 3 predicts and pickles in the
    # background, 4 exchanges the storage_meta part of 3's bytes; 5 plans anew, 6 is the first to predict again
    assert saver.wrote[:2] == ["object", "object"] and saver.wrote[2:4] == ["bytes", "bytes"]
    assert respliced[:2] == [False, True]
    assert saver.wrote[4] == "object" and respliced[2:] == ([False] if saver.wrote[5] == "bytes" else [])
