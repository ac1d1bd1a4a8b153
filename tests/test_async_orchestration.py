"""Plan / write / finish as separate calls (the sequence an async framework drives), on the CPU with the oracle's
saver: call order, plan caching across saves, results hand-over through the manager proxies.

Expectations follow the reference's tests of the same functions (tests/adapter/pytorch/test_custom_state_dict_saver.py
:60-454: cache validated on the second save and reused from the third; metadata None when the cached plan is reused)
and of the Megatron strategy's ordering (tests/adapter/megatron/test_save_strategies.py:160-456).
"""

import concurrent.futures
import os
import pickle

import pytest
import torch
import torch.multiprocessing as torch_mp
from torch.distributed.checkpoint import DefaultSavePlanner
from torch.distributed.checkpoint.utils import _DistWrapper

from ml_flashpoint.adapter.pytorch import custom_state_dict_saver as statedictsaver
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
from oracle import mlf_format as fmt
from oracle.cpu_path import OracleCheckpointSaver

pytestmark = pytest.mark.filterwarnings("ignore:torch.distributed is disabled")


@pytest.fixture(scope="module")
def manager_future():
    mgr = torch_mp.get_context("spawn").Manager()
    fut = concurrent.futures.Future()
    fut.set_result(mgr)
    yield fut
    mgr.shutdown()


class RecordingSaver(OracleCheckpointSaver):
    def __init__(self, log, **kw):
        super().__init__(**kw)
        self.log = log

    def initialize_checkpoint(self, cid):
        self.log.append("initialize_checkpoint")
        return super().initialize_checkpoint(cid)

    def prepare_write_data(self, *a, **kw):
        self.log.append("prepare_write_data")
        return super().prepare_write_data(*a, **kw)

    def write_data(self, *a, **kw):
        self.log.append("write_data")
        return super().write_data(*a, **kw)

    def write_metadata(self, *a, **kw):
        self.log.append("write_metadata")
        return super().write_metadata(*a, **kw)

    def finalize_checkpoint(self, cid):
        self.log.append("finalize_checkpoint")
        return super().finalize_checkpoint(cid)


def test_three_saves_validate_then_reuse_the_cached_plan(shm_dir, manager_future):
    log = []
    saver = RecordingSaver(log)
    dist = _DistWrapper(None, False, 0)  # single process: collectives are identities
    sd = {"w": torch.arange(12.0).reshape(3, 4), "b": torch.ones(5, dtype=torch.int64)}
    cached = None
    metadata_kept = None
    flags = []
    for step in (1, 2, 3):
        cid = CheckpointContainerId(os.path.join(shm_dir, f"step-{step}_ckpt"))
        log.clear()
        saver.initialize_checkpoint(cid)
        writer = MemoryStorageWriter(saver, manager_future)  # the strategy makes a fresh writer per save
        writer.reset(cid.data)
        sd["w"] += 1
        buckets, metadata, central, local, validated = statedictsaver.generate_plan(
            cid, sd, writer, DefaultSavePlanner(), dist, cached_ckpt_structure=cached
        )
        flags.append((validated, metadata is None))
        cached = (central, local, validated)
        metadata_kept = metadata or metadata_kept
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        results = statedictsaver.write_data(cid, writer, staged, replicate_after_write=False)
        assert writer.get_write_results(cid) == results
        statedictsaver.finish_write(cid, writer, metadata_kept, dist)
        saver.finalize_checkpoint(cid)
        assert log == ["initialize_checkpoint", "initialize_checkpoint", "prepare_write_data", "write_data",
                       "write_metadata", "finalize_checkpoint"]
        raw = open(os.path.join(cid.data, "__0__0_src0.distcp"), "rb").read()
        md = pickle.load(open(os.path.join(cid.data, ".metadata"), "rb"))
        order = [i.fqn for i, _ in sorted(md.storage_data.items(), key=lambda kv: kv[1].offset)]
        assert raw == fmt.file_image([sd[k] for k in order])[0]
        assert not os.path.exists(f"{cid}__0__unfinished")
    # 1st save: nothing cached.  2nd: the fresh central plan equals the cached one -> validated.  3rd: reused, so
    # neither the plan exchange nor the metadata broadcast ran.
    assert flags == [(False, False), (True, False), (True, True)]
