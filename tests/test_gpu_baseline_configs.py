"""The benchmark's configurations on their own workload generators, at sizes the CPU oracle finishes in seconds:
saved through ``dcp.save`` with the gfx950 saver, the object compared **byte for byte** with the oracle's file image,
then restored through ``dcp.load`` and compared bit for bit.

* 2 000 small tensors (64 B .. 4 MB log-uniform, fp32 / bf16 / int64) in one plan;
* 96 non-contiguous views (transposed blocks, every-other-column bands, 16-row blocks; bf16 / fp8-e4m3 / fp32) of
  three shared parents;
* a slice of the Mixtral expert shard (bf16 expert matrices, attention, router, norms);
* GPT-2-small at its full 124 M parameters, resident in **host** memory, written by the gfx950 saver into a **pooled**
  buffer (host tensors of this size go from host memory straight into the buffer).
"""

import concurrent.futures
import os
import pickle

import pytest
import torch
import torch.distributed.checkpoint as dcp

import workloads
from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.buffer_pool import BufferPoolConfig
from oracle import mlf_format as fmt

pytestmark = [pytest.mark.gpu, pytest.mark.filterwarnings("ignore:torch.distributed is disabled")]
DEV = "cuda:0"


class _LocalManager:
    def dict(self):
        return {}

    def Event(self):
        import threading

        return threading.Event()


@pytest.fixture
def manager_future():
    fut = concurrent.futures.Future()
    fut.set_result(_LocalManager())
    return fut


@pytest.fixture(autouse=True)
def _fresh_pool():
    CheckpointObjectManager._worker_pool = None
    yield
    CheckpointObjectManager().teardown_pool()


def _saver(manager=None, **kw):
    from ml_flashpoint.core.checkpoint_saver import DefaultMLFlashpointCheckpointSaver

    return DefaultMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, manager or CheckpointObjectManager(),
                                              None, initial_buffer_size_bytes=1 << 20, **kw)


def _loader(manager=None, **kw):
    from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader

    return DefaultMLFlashpointCheckpointLoader(manager or CheckpointObjectManager(), None, **kw)


def _bits(t):
    flat = t.detach().contiguous().cpu().reshape(-1)
    if flat.numel() and flat.stride(0) != 1:
        flat = flat.clone()
    return flat.view(torch.uint8)


def _save_compare_restore(sd, ckpt, manager_future, saver, loader):
    """dcp.save -> the object equals the oracle's image of the same tensors in the plan's order, offsets follow the
    reference's rules -> dcp.load into zeroed targets -> bit-exact.  Returns the object's bytes."""
    originals = {k: _bits(v) for k, v in sd.items()}
    host_copies = {k: v.detach().cpu() for k, v in sd.items()}  # same shapes and strides as the views they copy
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    assert sorted(n for n in os.listdir(ckpt) if not n.endswith(".crc32c")) == [".metadata", "__0__0_src0.distcp"]
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    by_offset = sorted(metadata.storage_data.items(), key=lambda kv: kv[1].offset)
    assert len(by_offset) == len(sd)
    want, spans = fmt.file_image([host_copies[i.fqn] for i, _ in by_offset])
    assert [(s.offset, s.length) for _, s in by_offset] == spans
    assert spans[0][0] == 0 and all(a[0] + a[1] == b[0] for a, b in zip(spans, spans[1:]))
    assert len(raw) == len(want)
    if raw != want:
        first = next(i for i, (a, b) in enumerate(zip(raw, want)) if a != b)
        pytest.fail(f"object differs from the oracle's image at file byte {first}")
    for v in sd.values():
        v.zero_() if v.is_contiguous() else v.fill_(0)
    dcp.load(sd, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    if torch.cuda.is_available():
        torch.cuda.synchronize()
    wrong = [k for k, v in sd.items() if not torch.equal(_bits(v), originals[k])]
    assert not wrong, wrong[:5]
    return raw


def test_many_small_tensors_in_one_plan(shm_dir, manager_future):
    sd = workloads.many_small(DEV, count=2000)
    assert len(sd) == 2000 and {t.dtype for t in sd.values()} == {torch.float32, torch.bfloat16, torch.int64}
    sizes = [t.numel() * t.element_size() for t in sd.values()]
    assert min(sizes) < 256 and max(sizes) > (2 << 20)  # both ends of the 64 B .. 4 MB range are present
    saver, loader = _saver(crc_chunk_bytes=1 << 20), _loader()
    _save_compare_restore(sd, os.path.join(shm_dir, "step-3_ckpt"), manager_future, saver, loader)
    assert loader.last_load_stats["device_items"] == 2000
    # a second save of the same tensors goes through the kept plan and writes the same bytes
    _save_compare_restore(sd, os.path.join(shm_dir, "step-4_ckpt"), manager_future, saver, loader)
    assert saver.last_save_stats.get("plans_reused") == 1


def test_strided_views_of_shared_parents(shm_dir, manager_future):
    sd, parents = workloads.strided_views(DEV, count=96, min_dim=256, max_dim=2048, mean_view_bytes=256 << 10)
    n_parents = len(parents)
    combos = {(t.dtype, (i // n_parents) % 3) for i, t in enumerate(sd.values())}
    assert len(combos) == 9  # bf16 / fp8-e4m3 / fp32 x transposed / every other column / row block
    assert sum(not t.is_contiguous() for t in sd.values()) >= 60
    from ml_flashpoint.hip import plan as P

    layout = P.build_save_layout(list(sd.values()))
    info = P.Plan(layout.items, layout.blob, layout.image_bytes).info
    assert info.n_transposed_items > 0 and info.n_strided_items > 0 and info.n_flat_tiles > 0  # all three kernels
    before = [p.clone() for p in parents]
    _save_compare_restore(sd, os.path.join(shm_dir, "step-5_ckpt"), manager_future, _saver(crc_chunk_bytes=1 << 20),
                          _loader())
    # bytes of the parents that no view covers were zeroed by nobody and written by nobody; those that views cover
    # came back: the parents are what they were
    assert all(torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(before, parents))


def test_mixtral_expert_shard_slice(shm_dir, manager_future):
    sd = workloads.mixtral_expert_shard(DEV, layers=2, experts=8, d=512, ffn=1792, kv=128)
    assert len(sd) == 2 * (7 + 8 * 3) and all(t.dtype == torch.bfloat16 for t in sd.values())
    _save_compare_restore(sd, os.path.join(shm_dir, "step-4_ckpt"), manager_future, _saver(crc_chunk_bytes=1 << 20),
                          _loader())


def test_gpt2_small_full_size_on_host_into_a_pooled_buffer(shm_dir, manager_future):
    """The CPU-runnable configuration as the benchmark words it: fp32 GPT-2-small in host memory through the DCP
    adapter into the shm buffer pool - with the product's saver, pool and BufferIO on the path."""
    sd = workloads.gpt2_small("cpu")
    assert len(sd) == 148 and sum(t.numel() for t in sd.values()) == 124_439_808
    manager = CheckpointObjectManager(BufferPoolConfig(os.path.join(shm_dir, "pool"), 0, 2, METADATA_SIZE + (1 << 20)))
    saver, loader = _saver(manager), _loader(manager)
    ckpt = os.path.join(shm_dir, "run", "step-1_ckpt")
    raw = _save_compare_restore(sd, ckpt, manager_future, saver, loader)
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    assert os.path.islink(obj) and os.path.dirname(os.readlink(obj)) == os.path.join(shm_dir, "pool")
    assert len(raw) == METADATA_SIZE + sum(len(fmt.record_bytes(t)) for t in sd.values())
    assert saver.last_save_stats.get("host_copy_bytes", 0) > 400e6  # the large tensors went host to buffer
    assert loader.last_load_stats["host_items"] == 148
    # the same state dict resident on the device gives the same file
    sd_dev = {k: v.to(DEV) for k, v in sd.items()}
    ckpt2 = os.path.join(shm_dir, "run", "step-2_ckpt")
    assert _save_compare_restore(sd_dev, ckpt2, manager_future, saver, loader) == raw
