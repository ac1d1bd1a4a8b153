"""Benchmark of the save/restore data path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3-8b-shard] [--scale S]

A *step* is one full save of the workload's state dict (resident in HBM) into a pooled tmpfs buffer object, followed
by one full restore of that object into the (zeroed) live tensors.  The save is the reference's three-call sequence
(``generate_plan`` -> stage -> ``write_data`` -> ``finish_write``, then ``finalize_checkpoint``) over
``MemoryStorageWriter``; the restore is ``dcp.load`` over ``MemoryStorageReader``; the gfx950 saver/loader are plugged
in, CRC-32C per 32 MiB chunk is computed on save and verified on restore.  Prints ONE JSON line:

* ``value``          GB/s moved through the path per step: (bytes saved + bytes restored) / step time
* ``save_GBps`` / ``restore_GBps`` / ``blocking_save_ms`` (save entry -> training stream may continue) and the
  stage breakdown (pack / unpack kernel GB/s from HIP events, D2H / H2D GB/s of the copy engine)
* ``roofline``       the pack kernel against HBM peak: algorithmic bytes = 2 x payload bytes per launch
* ``cpu_baseline``   the CPU oracle (restating the reference's per-tensor path) timed on this box's host cores on a
                     bounded sample of the same state dict

Synthetic data, seeded; the restored tensors are checked against fingerprints of the originals after the timed region.
"""

import argparse
import concurrent.futures
import gc
import json
import os
import shutil
import sys
import tempfile
import time

REPO = os.path.dirname(os.path.abspath(__file__))
for _p in (REPO, os.path.join(REPO, "ml-flashpoint_amd"), os.path.join(REPO, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, vendor figure
# HBM bytes moved by one pack, relative to its algorithmic bytes (2 x payload), by (workload, where the checksums are
# computed): measured with `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`, each scaled against a torch.add kernel of
# known size (summaries: profiles/pmc_traffic_*.md).  Hardware counters cannot be read from inside this script, so the
# ratio of the same workload at full scale is applied to the live algorithmic byte count; other runs report null.
PACK_TRAFFIC_RATIO = {
    ("llama3-8b-shard", "beside"): 1.0008,
    ("llama3-8b-shard", "fused"): 1.0158,
    ("strided-views", "beside"): 1.214,
    ("mixtral-expert-shard", "beside"): 1.0008,
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="llama3-8b-shard",
                    choices=["llama3-8b-shard", "many-small", "mixtral-expert-shard", "strided-views", "gpt2-small",
                             "offloaded-optimizer"])
    ap.add_argument("--scale", type=float, default=1.0, help="fraction of the workload's layers/tensors (debugging)")
    ap.add_argument("--tile-bytes", type=int, default=0)
    ap.add_argument("--block-threads", type=int, default=0)
    ap.add_argument("--slot-mib", type=int, default=32)
    ap.add_argument("--slots", type=int, default=3)
    ap.add_argument("--copy-threads", type=int, default=0, help="0 = the engine's default (CPUs available, at most 16)")
    ap.add_argument("--crc-chunk-mib", type=int, default=32,
                    help="CRC-32C per chunk of this size, computed on the GPU during the save and verified on the GPU during "
                         "the restore (0 = off)")
    ap.add_argument("--save-crc", choices=["beside", "fused", "host"], default="host",
                    help="where the save's checksums are computed: a pass of its own beside the transfer, inside the pack "
                         "kernel, or by the host threads that move the pinned slots into the buffer")
    ap.add_argument("--restore-crc", choices=["fused", "before"], default="before",
                    help="how the restore verifies them: a pass over every uploaded window before it is unpacked (the "
                         "loader's default), or inside the unpack kernel")
    ap.add_argument("--cpu-baseline-gb", type=float, default=12.0, help="size of the CPU baseline's sample (0 = skip)")
    ap.add_argument("--plan-cache", action="store_true",
                    help="reuse the save plan across steps once two consecutive plans compared equal, as the reference's "
                         "async strategy does (off: every step plans from scratch, like dcp.save)")
    ap.add_argument("--save-io", choices=["mmap", "file"], default="mmap", help="host side of the save: memcpy into the mapping, or pwrite")
    ap.add_argument("--restore-io", choices=["mmap", "file"], default="file", help="host side of the restore: read the mapping, or pread")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one plain elementwise kernel (torch.add, 4 GiB in, 4 GiB out) so that hardware byte "
                         "counters of a profiler run can be scaled against a kernel of known traffic")
    ap.add_argument("--partial-restore-prefix", default=None,
                    help="after the timed steps, also time a restore of only the entries whose names start with this "
                         "(e.g. 'model.': the weights out of weights + optimizer state); reported as partial_restore")
    ap.add_argument("--max-image-gb", type=float, default=0.0,
                    help="cap on the image held in HBM at once (saver and loader): smaller than the object, the save "
                         "goes window by window and blocks for the transfer; 0 = what the device has free")
    ap.add_argument("--whole-image-restore", action="store_true",
                    help="restore through one device buffer for the whole object instead of two alternating ones")
    ap.add_argument("--no-prefault", action="store_true", help="leave the pool file's pages to the first save, as the reference does")
    ap.add_argument("--no-link-probe", action="store_true", help="skip the bare host-link and device-copy measurements")
    ap.add_argument("--no-busy-gpu-probe", action="store_true",
                    help="skip the save whose transfer runs on a background thread while bf16 GEMMs, then HBM copies, keep "
                         "the device busy (what the transfer costs them, and what they cost the transfer)")
    ap.add_argument("--no-crc-compare", action="store_true", help="skip the extra saves in the other checksum mode")
    ap.add_argument("--no-plan-cache-compare", action="store_true", help="skip the extra saves on a reused DCP plan")
    ap.add_argument("--no-limited-hbm-compare", dest="limited_hbm_compare", action="store_false",
                    help="skip the extra save + restore with room in HBM for 57 %% and for 14 %% of the image")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="the default run (llama3-8b-shard at full scale) also measures the many-small and strided-views "
                         "configurations, one warm-up and three timed steps each, and reports them under other_workloads")
    ap.add_argument("--root", default=None, help="directory on tmpfs for the pool and checkpoints")
    return ap.parse_args()


def build_workload(name, device, scale):
    import workloads

    if name == "llama3-8b-shard":
        layers = max(1, round(32 * scale))
        sd = workloads.llama3_8b_shard(device, layers=layers) if scale >= 1.0 else workloads.llama3_8b_shard(
            device, layers=layers, vocab=max(1024, int(128256 * scale)))
        label = "Llama-3-8B-shaped shard: bf16 weights + fp32 master + fp32 Adam m,v"
    elif name == "many-small":
        sd = workloads.many_small(device, count=max(1, int(20000 * scale)))
        label = "20,000 tensors, 64 B..4 MB log-uniform, fp32/bf16/int64"
    elif name == "mixtral-expert-shard":
        sd = workloads.mixtral_expert_shard(device, layers=max(1, round(32 * scale)))
        label = "Mixtral-8x7B-shaped expert shard, bf16"
    elif name == "strided-views":
        sd, parents = workloads.strided_views(device, count=max(3, int(2000 * scale)))
        sd = dict(sd)
        sd["__parents__"] = parents  # keep alive; not a tensor entry
        label = "2,000 transposed / strided / row-block views of bf16/fp8/fp32 parents"
    elif name == "offloaded-optimizer":
        sd = workloads.offloaded_optimizer_shard(device, layers=max(1, round(8 * scale)))
        label = "bf16 weights on the device, fp32 master + Adam m,v in host memory"
    else:
        sd = workloads.gpt2_small(device)
        label = "GPT-2-small fp32"
    parents = sd.pop("__parents__", None)
    return sd, label, parents


def cpu_baseline(sd, sample_bytes, root, device, passes=5):
    """The reference's CPU path, restated by the oracle, on a prefix of the state dict of about ``sample_bytes``
    (the whole of it when that is larger)."""
    import torch

    from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
    from oracle import cpu_path

    sample, total = {}, 0
    for k, v in sd.items():
        if total >= sample_bytes:
            break
        sample[k] = v
        total += v.numel() * v.element_size()
    capacity = total + 256 * len(sample) + (1 << 20)  # payloads + record headers (~140 B each) + slack
    saver = cpu_path.OracleCheckpointSaver(initial_buffer_size_bytes=capacity)
    threads = saver.torch_thread_count(1)
    cid = CheckpointContainerId(os.path.join(root, "cpu_baseline", "step-0_ckpt"))
    path = os.path.join(cid.data, "sample.distcp")
    tensors = list(sample.values())
    times = {"stage": [], "write": [], "restore": []}
    for rep in range(1 + passes):  # the first pass faults the tmpfs pages in, like the GPU path's prime iteration
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        staged = saver.stage_data(cid, sample, non_blocking=True)
        t1 = time.perf_counter()
        original = torch.get_num_threads()
        torch.set_num_threads(threads)
        try:
            if rep == 0:
                spans = cpu_path.write_object(path, list(staged.values()), [], capacity)
                t2 = time.perf_counter()
            else:
                # rewrite in place over warm pages: what a pooled buffer gives the reference from the second save on
                spans = _rewrite_warm(path, list(staged.values()))
                t2 = time.perf_counter()
        finally:
            torch.set_num_threads(original)
        del staged
        # restore: read() copy, frombuffer, copy_ to the device tensor
        import mmap

        from oracle import mlf_format as fmt

        targets = [torch.empty_like(t) for t in tensors]
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        with open(path, "rb") as f:
            mm = mmap.mmap(f.fileno(), 0, mmap.MAP_SHARED, mmap.PROT_READ)
            for (off, length), tgt in zip(spans, targets):
                record = mm[fmt.METADATA_SIZE + off : fmt.METADATA_SIZE + off + length]
                tgt.copy_(fmt.read_item(record, (0,) * tgt.dim(), tuple(tgt.shape)))
            mm.close()
        torch.cuda.synchronize()
        t4 = time.perf_counter()
        ok = all(torch.equal(a.view(torch.uint8), b.contiguous().view(torch.uint8)) for a, b in zip(targets[:8], tensors[:8]))
        del targets
        if rep:  # the warm-up pass is not counted
            times["stage"].append(t1 - t0)
            times["write"].append(t2 - t1)
            times["restore"].append(t4 - t3)
    shutil.rmtree(os.path.join(root, "cpu_baseline"), ignore_errors=True)
    import statistics

    stage, write, restore = (statistics.median(times[k]) for k in ("stage", "write", "restore"))
    gb = total / 1e9
    return {
        "value": round(2 * gb / (stage + write + restore), 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": (f"all {len(sample)} tensors" if len(sample) == len(sd) else f"first {len(sample)} tensors") +
                  f" ({gb:.2f} GB) of the same state dict; one warm-up pass, then the median of {passes} (warm tmpfs pages)",
        "tensors": len(sample),
        # the reference's per-tensor loops: stage (.to("cpu")), write (header + copy_ into the mapping), restore
        "us_per_tensor": {"stage": round(stage * 1e6 / len(sample), 1), "write": round(write * 1e6 / len(sample), 1),
                          "restore": round(restore * 1e6 / len(sample), 1)},
        "passes": passes,
        "spread": {k: [round(min(v), 3), round(max(v), 3)] for k, v in times.items()},
        "save_GBps": round(gb / (stage + write), 3),
        "restore_GBps": round(gb / restore, 3),
        "blocking_stage_ms": round(stage * 1e3, 1),
        "write_GBps": round(gb / write, 3),
        "host_cpus": os.cpu_count(),
        "usable_cpus": len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else None,
        "numa_nodes_online": _read_text("/sys/devices/system/node/online"),
        "tmpfs_root": root,
        "restored_ok": bool(ok),
    }


def _read_text(path):
    try:
        with open(path) as f:
            return f.read().strip()
    except OSError:
        return None


def _rewrite_warm(path, tensors):
    """Second write of the CPU baseline: same records into the already-populated file (no truncation)."""
    import mmap

    import torch

    from oracle import mlf_format as fmt

    spans, pos = [], 0
    with open(path, "r+b") as f:
        mm = mmap.mmap(f.fileno(), 0, mmap.MAP_SHARED, mmap.PROT_READ | mmap.PROT_WRITE)
        mv = memoryview(mm)
        for t in tensors:
            start = pos
            hdr = fmt.header_bytes(fmt.dtype_name(t.dtype), tuple(t.shape))
            mv[fmt.METADATA_SIZE + pos : fmt.METADATA_SIZE + pos + len(hdr)] = hdr
            pos += len(hdr)
            nbytes = t.numel() * t.element_size()
            if nbytes:
                dest = mv[fmt.METADATA_SIZE + pos : fmt.METADATA_SIZE + pos + nbytes]
                torch.frombuffer(dest, dtype=t.dtype, count=t.numel()).reshape(t.shape).copy_(t)
                del dest
                pos += nbytes
            spans.append((start, pos - start))
        mv.release()
        mm.close()
    return spans


def _hbm_copy_probe(device, tile_bytes, block_threads, nbytes=8 << 30, reps=5):
    """What this device's memory gives a plain copy, measured in the same run as the pack: torch's device-to-device
    ``copy_`` of ``nbytes``, and this library's flat kernel packing one contiguous tensor of that size (one record
    header, one span, no other tables).  Both move 2 x ``nbytes``; the best of ``reps`` launches counts."""
    import torch

    from ml_flashpoint.hip import plan as hip_plan

    src = torch.zeros(nbytes, dtype=torch.uint8, device=device)
    layout = hip_plan.build_save_layout([src])
    image = torch.empty(layout.image_bytes, dtype=torch.uint8, device=device)
    plan = hip_plan.Plan(layout.items, layout.blob, layout.image_bytes, tile_bytes=tile_bytes, block_threads=block_threads)
    stream = torch.cuda.current_stream(device)

    def best_ms(launch):
        launch()  # untimed first launch
        times = []
        for _ in range(reps):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record(stream)
            launch()
            end.record(stream)
            end.synchronize()
            times.append(begin.elapsed_time(end))
        return min(times)

    try:
        torch_ms = best_ms(lambda: image[:nbytes].copy_(src))
        flat_ms = best_ms(lambda: plan.pack(image, stream.cuda_stream))
    finally:
        plan.destroy()
    return {"bytes": nbytes, "torch_copy_GBps": round(2 * nbytes / 1e6 / torch_ms, 1),
            "flat_kernel_one_tensor_GBps": round(2 * nbytes / 1e6 / flat_ms, 1),
            "what": "read + write rate of a device-to-device copy of one contiguous tensor: torch's copy_ and this "
                    "library's pack kernel, best of %d launches each" % reps}


def _busy_gpu_probe(device, saver, sd, root, manager):
    """One save with ``background_write=True`` (the transfer starts inside ``prepare_write_data`` on a thread) while
    this thread keeps the device busy the way a training step would: 8192^3 bf16 GEMMs for the first half of the
    transfer, 4 GiB device-to-device copies for the second.  Returns their rates alone and beside the transfer, and
    how long the save took."""
    import torch
    from torch.distributed.checkpoint.planner_helpers import _create_write_items

    from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId

    torch.cuda.empty_cache()  # (or the operands below would be cut out of the block the images of the steps lay in)
    a = torch.randn(8192, 8192, device=device, dtype=torch.bfloat16)
    b = torch.randn(8192, 8192, device=device, dtype=torch.bfloat16)
    x = torch.empty(1 << 30, dtype=torch.float32, device=device)
    y = torch.empty_like(x)

    def gemms(seconds):
        torch.cuda.synchronize()
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(20):
                torch.matmul(a, b)
            torch.cuda.synchronize()
            n += 20
        return n * 2 * 8192 ** 3 / (time.perf_counter() - t0) / 1e12

    def copies(seconds):
        torch.cuda.synchronize()
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(10):
                y.copy_(x)
            torch.cuda.synchronize()
            n += 10
        return n * 2 * x.numel() * 4 / (time.perf_counter() - t0) / 1e12

    class Resolver:
        def resolve_data(self, item):
            return sd[item.index.fqn]

    gemms(0.5)  # clocks up
    alone = (gemms(1.0), copies(1.0))
    items = [wi for k, v in sd.items() if isinstance(v, torch.Tensor) for wi in _create_write_items(k, v)]
    out = None
    for step in range(2):  # the second runs on the kept plan
        cid = CheckpointContainerId(os.path.join(root, "run", f"step-{3000 + step}_ckpt"))
        t0 = time.perf_counter()
        buckets = saver.prepare_write_data(cid, items, Resolver(), "busy", 1)
        beside = (gemms(0.8), copies(0.8))
        saver.write_data(cid, buckets, replicate_after_write=False, thread_count=1)
        out = {"save_s": round(time.perf_counter() - t0, 3),
               "gemm_TFLOPs": {"alone": round(alone[0], 1), "beside_the_transfer": round(beside[0], 1)},
               "hbm_copy_TBps": {"alone": round(alone[1], 3), "beside_the_transfer": round(beside[1], 3)}}
        manager.delete_container(cid)
    saver.release_device_memory()
    return out


class _LocalManager:
    """In-process stand-in for ``torch.multiprocessing.Manager()``: ``dict()`` and ``Event()`` only."""

    def dict(self):
        return {}

    def Event(self):
        import threading

        return threading.Event()

    def shutdown(self):
        pass


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the save/restore path; runs with --gpus > 1 are not part of this "
              "build (each rank would run this same pipeline independently on its own shard).", file=sys.stderr)
        sys.exit(2)
    result = run_workload(args)
    if args.workload == "llama3-8b-shard" and args.scale >= 1.0 and args.max_image_gb <= 0 and not args.no_other_workloads:
        # the configurations whose cost is not in the bytes: 20 000 small tensors (host time per tensor) and 2 000
        # non-contiguous views (gather / transpose / scatter kernels); same pipeline, fewer steps, no side probes
        keep = ("save_GBps", "restore_GBps", "blocking_save_ms", "blocking_breakdown_ms", "blocking_host_us_per_tensor",
                "save_tail_ms", "pack_GBps", "unpack_GBps", "unpack_GBps_beside_h2d", "d2h_GBps", "h2d_GBps",
                "restore_breakdown_ms", "with_dcp_plan_cache", "cpu_baseline", "parity", "ms_per_step", "value")
        others = {}
        for name in ("many-small", "strided-views"):
            sub = argparse.Namespace(**vars(args))
            sub.workload, sub.steps, sub.warmup = name, 3, 1
            sub.no_link_probe = sub.no_crc_compare = sub.no_busy_gpu_probe = True
            sub.limited_hbm_compare = False
            sub.partial_restore_prefix, sub.pmc_calibration = None, False
            sub.no_plan_cache_compare = name != "many-small"  # where the DCP planner is most of the blocking time
            sub.cpu_baseline_gb = 1e3 if name == "many-small" and args.cpu_baseline_gb > 0 else 0.0  # the whole dict
            sub.cpu_baseline_passes = 3
            full = run_workload(sub)
            others[name] = {"workload": full["config"]["workload"], "tensors": full["config"]["tensors"],
                            "payload_bytes": full["config"]["payload_bytes"], "steps": sub.steps, "warmup": sub.warmup,
                            **{k: full[k] for k in keep if k in full},
                            "pack_frac_of_hbm_peak": full["roofline"]["frac"], "pack_ms": full["roofline"]["avg_launch_ms"]}
        result["other_workloads"] = others
    print(json.dumps(result), flush=True)


def run_workload(args):
    """Builds the workload, runs the prime, warm-up and timed steps and the side measurements the arguments ask for,
    gives the device memory back and returns the result line as a dict."""
    import torch
    import torch.distributed.checkpoint as dcp
    from torch.distributed.checkpoint import DefaultSavePlanner

    import workloads
    from torch.distributed.checkpoint.utils import _DistWrapper

    from ml_flashpoint.adapter.pytorch import custom_state_dict_saver as state_dict_saver
    from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
    from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.core.buffer_pool import BufferPoolConfig
    from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
    from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader
    from ml_flashpoint.core.checkpoint_saver import DefaultMLFlashpointCheckpointSaver
    from ml_flashpoint.hip.checkpoint_saver import EngineConfig

    import warnings

    warnings.filterwarnings("ignore", message="torch.distributed is disabled")
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    t_setup = time.perf_counter()
    sd, label, parents = build_workload(args.workload, device, args.scale)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    payload = workloads.payload_bytes(sd)
    prints = {k: workloads.fingerprint(v) for k, v in sd.items()}
    torch.cuda.synchronize()
    print(f"[bench] workload {args.workload}: {len(sd)} tensors, {payload / 1e9:.2f} GB payload, built in "
          f"{time.perf_counter() - t_setup:.1f}s", file=sys.stderr, flush=True)

    base = args.root or ("/dev/shm" if os.access("/dev/shm", os.W_OK) else None)
    root = tempfile.mkdtemp(prefix="mlf_bench_", dir=base)
    # the writer keeps its per-checkpoint results in Manager proxies so that a worker *process* can fill them in;
    # this benchmark runs the whole save in one process, so an in-process stand-in with the same two factory
    # methods is enough (and keeps a helper process out of the profile)
    mgr = _LocalManager()
    fut = concurrent.futures.Future()
    fut.set_result(mgr)
    engine_cfg = EngineConfig(slot_bytes=args.slot_mib << 20, n_slots=args.slots, copy_threads=args.copy_threads)
    # one pooled buffer of the object's size (payload + record headers + slack), created before the first save the
    # way a job creates its pool at start-up: its pages are allocated and mapped on a background thread
    # (BufferPoolConfig.prefault), and the previous step's object is deleted before the next save, as
    # finalize_checkpoint's background cleanup would have done, so the same pages are reused every step
    CheckpointObjectManager._worker_pool = None
    pool_bytes = METADATA_SIZE + payload + 256 * len(sd) + (1 << 20)
    manager = CheckpointObjectManager(BufferPoolConfig(os.path.join(root, "pool"), 0, 1, pool_bytes,
                                                       prefault=not args.no_prefault))
    t_pool = time.perf_counter()
    manager.warm_up_pool()
    max_image = int(args.max_image_gb * 1e9) if args.max_image_gb > 0 else None

    def make_saver(crc_mode, **more):
        made = DefaultMLFlashpointCheckpointSaver(
            lambda: 0, lambda: 0, lambda: None, manager, None, initial_buffer_size_bytes=1 << 20,
            engine_config=engine_cfg, tile_bytes=args.tile_bytes, block_threads=args.block_threads,
            crc_chunk_bytes=args.crc_chunk_mib << 20, crc_mode=crc_mode, use_file_io=args.save_io == "file",
            max_image_bytes=more.pop("max_image_bytes", max_image), **more)
        made.record_kernel_events = True
        return made

    saver = make_saver(args.save_crc)
    saver.warm_up(device)  # at start-up, like the pool: pinned slots, streams clear of the training stream's queue
    loader = DefaultMLFlashpointCheckpointLoader(manager, None, engine_config=engine_cfg, tile_bytes=args.tile_bytes,
                                                 block_threads=args.block_threads, use_file_io=args.restore_io == "file",
                                                 crc_mode=args.restore_crc, max_image_bytes=max_image,
                                                 pipelined_restore=not args.whole_image_restore)
    loader.record_kernel_events = True
    result = None
    if args.pmc_calibration:
        cal_src = torch.ones(1 << 30, dtype=torch.float32, device=device)
        cal_dst = torch.empty_like(cal_src)
        torch.add(cal_src, 1.0, out=cal_dst)  # reads 4 GiB, writes 4 GiB
        torch.cuda.synchronize()
        del cal_src, cal_dst
        torch.cuda.empty_cache()
    dist = _DistWrapper(None, False, 0)
    state = {"cached": None, "metadata": None, "use_cache": args.plan_cache}

    def one_save(the_saver, cid):
        """The reference's three-call form of a save (plan / write / finish), as its async strategy drives it.
        Returns the wall times of its parts; the blocking part ends where the training stream may go on."""
        the_saver.kernel_events.clear()
        gc.collect()  # outside the timed regions: a full collection of this process's heap takes ~60 ms
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        the_saver.initialize_checkpoint(cid)
        writer = MemoryStorageWriter(the_saver, fut)
        writer.reset(cid.data)
        buckets, md, central, local, validated = state_dict_saver.generate_plan(
            cid, sd, writer, DefaultSavePlanner(), dist, state["cached"] if state["use_cache"] else None)
        state["metadata"] = md if md is not None else state["metadata"]
        state["cached"] = (central, local, validated)
        if md is None:  # a cached plan: the caller holds the metadata object that goes with it
            writer.expect_metadata(state["metadata"])
        t_launch = time.perf_counter()
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        t_block = time.perf_counter()
        prepare_s = the_saver.last_save_stats.get("prepare_s", 0.0)
        results = state_dict_saver.write_data(cid, writer, staged, replicate_after_write=False)
        t_written = time.perf_counter()
        state_dict_saver.finish_write(cid, writer, state["metadata"], dist)
        the_saver.finalize_checkpoint(cid)
        t_saved = time.perf_counter()
        stats = dict(the_saver.last_save_stats)
        del buckets, staged, results
        return {"save": t_saved - t0, "blocking": t_block - t0, "plan": t_launch - prepare_s - t0, "pack_launch": prepare_s,
                "tail": t_saved - t_written, "write": t_written - t_block, "stats": stats,
                "metadata": ("previous bytes, storage_meta exchanged" if writer.early_metadata_respliced else
                             "pickled beside the transfer" if writer.early_metadata_used else "pickled in finish_write"),
                "pack_ms": sum(b.elapsed_time(e) for b, e, _ in the_saver.kernel_events),
                "pack_bytes": sum(n for _, _, n in the_saver.kernel_events)}

    try:
        rec = {}
        file_bytes = 0
        prev = None
        first = {}
        pool_prefault_s = manager.warm_up_pool(wait=True)
        pool_age_s = time.perf_counter() - t_pool
        # iteration 0 ("prime") is the first save and the first restore of the job; with the pool file's pages in
        # place it runs like any other, without them it pays for their allocation (~5 GB/s).  It is reported as
        # first_save_s / first_restore_s and not counted among the W warm-up and K timed steps.
        for it in range(1 + args.warmup + args.steps):
            timed = it >= 1 + args.warmup
            cid = CheckpointContainerId(os.path.join(root, "run", f"step-{it}_ckpt"))
            if prev is not None:
                manager.delete_container(prev)
            loader.kernel_events.clear()
            sv = one_save(saver, cid)
            d2h = sv["stats"]
            # ---- restore into zeroed live tensors ----
            for v in sd.values():
                v.zero_() if v.is_contiguous() else v.fill_(0)
            gc.collect()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            dcp.load(sd, checkpoint_id=cid.data, storage_reader=MemoryStorageReader(cid.data, loader), no_dist=True)
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            ld = dict(loader.last_load_stats)
            unpack_ms = sum(b.elapsed_time(e) for b, e, _ in loader.kernel_events)
            unpack_bytes = sum(n for _, _, n in loader.kernel_events)
            file_bytes = os.path.getsize(os.path.join(cid.data, "__0__0_src0.distcp"))
            prev = cid
            line = (f"[bench] it {it} {'timed ' if timed else ('prime ' if it == 0 else 'warmup')} save {sv['save']:.3f}s (blocking "
                    f"{sv['blocking'] * 1e3:.1f} ms, pack kernel {sv['pack_ms']:.2f} ms, d2h {d2h.get('d2h_s', 0):.3f}s, of which "
                    f"{d2h.get('d2h_wait_s', 0):.3f}s waiting for the pack) restore {t2 - t1:.3f}s (h2d {ld.get('h2d_s', 0):.3f}s, "
                    f"of which {ld.get('h2d_host_s', 0):.3f}s filling slots, unpack {unpack_ms:.2f} ms)")
            print(line, file=sys.stderr, flush=True)
            if it == 0:
                first = {"save": sv["save"], "restore": t2 - t1, "blocking": sv["blocking"]}
            if timed:
                row = {"step": sv["save"] + (t2 - t1), "save": sv["save"], "restore": t2 - t1, "blocking": sv["blocking"],
                       "plan": sv["plan"], "pack_launch": sv["pack_launch"], "save_tail": sv["tail"],
                       "d2h": d2h.get("d2h_s", 0.0), "d2h_bytes": d2h.get("d2h_bytes", 0),
                       "host_copy_s": d2h.get("host_copy_s", 0.0), "host_copy_bytes": d2h.get("host_copy_bytes", 0),
                       "h2d": ld.get("h2d_s", 0.0), "h2d_bytes": ld.get("h2d_bytes", 0), "h2d_host": ld.get("h2d_host_s", 0.0),
                       "pack_ms": sv["pack_ms"], "unpack_ms": unpack_ms, "pack_bytes": sv["pack_bytes"], "unpack_bytes": unpack_bytes,
                       "r_read": ld.get("read_s", 0.0), "r_parse": ld.get("parse_s", 0.0), "r_table": ld.get("table_s", 0.0),
                       "r_crc": ld.get("crc_s", 0.0), "r_unpack_plan": ld.get("unpack_plan_s", 0.0),
                       "r_plan_beside": ld.get("unpack_plan_beside_h2d_s", 0.0), "r_windows": ld.get("windows", 0),
                       "r_unpack": ld.get("unpack_s", 0.0), "r_commit": ld.get("commit_s", 0.0),
                       "r_early": ld.get("upload_began_before_parse", 0),
                       "windows": d2h.get("windows", 0), "image_pieces": d2h.get("image_pieces", 0)}
                for k, v in row.items():
                    rec.setdefault(k, []).append(v)
        # parity after the timed region: restored bits == original bits
        mismatched = [k for k, v in sd.items() if workloads.fingerprint(v) != prints[k]]
        assert not mismatched, f"restored tensors differ from the originals: {mismatched[:5]}"
        partial = None
        if args.partial_restore_prefix:
            subset = {k: v for k, v in sd.items() if k.startswith(args.partial_restore_prefix)}
            assert subset and len(subset) < len(sd), "--partial-restore-prefix must select some, not all, entries"
            times = []
            for _ in range(3):
                for v in subset.values():
                    v.zero_() if v.is_contiguous() else v.fill_(0)
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                dcp.load(subset, checkpoint_id=prev.data, storage_reader=MemoryStorageReader(prev.data, loader), no_dist=True)
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t1)
            assert all(workloads.fingerprint(v) == prints[k] for k, v in subset.items()), "partial restore differs"
            stats = loader.last_load_stats
            partial = {"prefix": args.partial_restore_prefix, "entries": len(subset),
                       "payload_bytes": workloads.payload_bytes(subset), "seconds": round(min(times), 4),
                       "uploaded_bytes": stats.get("h2d_bytes", 0), "ranges": stats.get("partial_read_ranges", 1)}
            print(f"[bench] partial restore of '{args.partial_restore_prefix}*': {partial}", file=sys.stderr, flush=True)

        mean = lambda xs: sum(xs) / len(xs)  # noqa: E731
        pack_s = mean(rec["pack_ms"]) * 1e-3
        algorithmic = 2 * mean(rec["pack_bytes"])
        # ---- the unpack kernels by themselves: one more restore through one image, nothing beside them ----
        clean_unpack = None
        if not args.whole_image_restore and max_image is None and mean(rec["r_windows"]) > 0:
            whole = DefaultMLFlashpointCheckpointLoader(manager, None, engine_config=engine_cfg, tile_bytes=args.tile_bytes,
                                                        block_threads=args.block_threads, use_file_io=args.restore_io == "file",
                                                        crc_mode=args.restore_crc, pipelined_restore=False)
            whole.record_kernel_events = True
            dcp.load(sd, checkpoint_id=prev.data, storage_reader=MemoryStorageReader(prev.data, whole), no_dist=True)
            torch.cuda.synchronize()
            clean_unpack = (sum(b.elapsed_time(e) for b, e, _ in whole.kernel_events) * 1e-3,
                            sum(n for _, _, n in whole.kernel_events))
            whole_engine = getattr(whole, "_engine", None)
            if whole_engine is not None:
                whole_engine.destroy()
            del whole

        # ---- the other way to the checksums, for comparison: two more saves (the first builds its plan) ----
        crc_modes = None
        if args.crc_chunk_mib and not args.no_crc_compare and max_image is None:
            image_bytes = file_bytes - METADATA_SIZE
            from ml_flashpoint.hip.integrity import read_sidecar
            import numpy as np
            reference_crcs = read_sidecar(os.path.join(prev.data, "__0__0_src0.distcp"))[2]
            crc_modes = {args.save_crc: {"pack_ms": round(pack_s * 1e3, 3), "blocking_save_ms": round(mean(rec["blocking"]) * 1e3, 2),
                                         "save_s": round(mean(rec["save"]), 4)}}
            for n_mode, other_mode in enumerate(m for m in ("beside", "fused", "host") if m != args.save_crc):
                other = make_saver(other_mode)
                runs = []
                for k in range(3):  # the first builds its plan and its engine
                    manager.delete_container(prev)
                    prev = CheckpointContainerId(os.path.join(root, "run", f"step-{1000 + 10 * n_mode + k}_ckpt"))
                    runs.append(one_save(other, prev))
                crc_modes[other_mode] = {"pack_ms": round(runs[-1]["pack_ms"], 3),
                                         "blocking_save_ms": round(runs[-1]["blocking"] * 1e3, 2),
                                         "save_s": round(min(r["save"] for r in runs[1:]), 4)}
                other.release_device_memory()
                if read_sidecar is not None:  # whoever computed them, the values are the same
                    crc_modes[other_mode]["same_checksums_as_" + args.save_crc] = bool(np.array_equal(
                        read_sidecar(os.path.join(prev.data, "__0__0_src0.distcp"))[2], reference_crcs))
            for mode, entry in crc_modes.items():
                # what one save moves through HBM: the pack reads and writes the payload, a checksum pass of its own
                # reads the image once more, the copies to the host read it once
                entry["save_hbm_bytes"] = {"pack": int(algorithmic), "checksum_pass": image_bytes if mode == "beside" else 0,
                                           "transfer_read": image_bytes}
                entry["save_hbm_bytes"]["total"] = sum(entry["save_hbm_bytes"].values())
        # ---- the same save once the plan of the previous one is reused (the reference's cached_ckpt_structure) ----
        with_cache = None
        if not args.plan_cache and not args.no_plan_cache_compare and max_image is None:
            state["use_cache"], runs = True, []
            for k in range(4):  # the first compares its plan with the last one's, the next ones skip the planning
                manager.delete_container(prev)
                prev = CheckpointContainerId(os.path.join(root, "run", f"step-{2000 + k}_ckpt"))
                runs.append(one_save(saver, prev))
            state["use_cache"] = False
            last, st = runs[-1], runs[-1]["stats"]
            part = lambda key: round(st.get(key, 0.0) * 1e3, 2)  # noqa: E731
            with_cache = {"blocking_save_ms": round(last["blocking"] * 1e3, 2), "dcp_plan_ms": round(last["plan"] * 1e3, 2),
                          "save_s": round(last["save"], 4), "metadata_object": last["metadata"],
                          # where the save's time goes: the blocking part (plan, layout + pack launch, the wait for the
                          # pack), then write_data (buffer acquired and sized, the transfer, close + truncate, the
                          # checksum sidecar, one WriteResult per item; the rest is the writer's own bookkeeping and
                          # the prediction of the results for the early metadata), then the tail (finish_write,
                          # finalize)
                          "save_breakdown_ms": {
                              "dcp_plan": round(last["plan"] * 1e3, 2), "layout_and_pack_launch": round(last["pack_launch"] * 1e3, 2),
                              "wait_for_pack": round((last["blocking"] - last["plan"] - last["pack_launch"]) * 1e3, 2),
                              "write_data": round(last["write"] * 1e3, 2), "of_write_acquire_buffer": part("acquire_s"),
                              "of_write_transfer": part("d2h_s"), "of_write_close_buffer": part("close_s"),
                              "of_write_sidecar": part("sidecar_s"), "of_write_results": part("results_s"),
                              "of_write_other": round((last["write"] - sum(st.get(k, 0.0) for k in (
                                  "acquire_s", "d2h_s", "close_s", "sidecar_s", "results_s"))) * 1e3, 2),
                              "tail_finish_and_finalize": round(last["tail"] * 1e3, 2)}}
        manager.delete_container(prev)

        # ---- the same object with room in HBM for part of its image only: the end of the object stays resident, the
        # rest goes window by window inside the blocking part; the restore goes through windows of that size ----
        limited = None
        if args.limited_hbm_compare and max_image is None and payload >= (8 << 30):
            limited = {}
            for share in (0.57, 0.14):  # 64 GB and 16 GB of room for the 112 GB shard
                room = int(payload * share)
                tight = make_saver(args.save_crc, max_image_bytes=room)
                tight_loader = DefaultMLFlashpointCheckpointLoader(
                    manager, None, engine_config=engine_cfg, tile_bytes=args.tile_bytes, block_threads=args.block_threads,
                    use_file_io=args.restore_io == "file", crc_mode=args.restore_crc, max_image_bytes=room)
                for again in range(2):  # the first creates the engines, their pinned slots and the window buffers
                    cid = CheckpointContainerId(os.path.join(root, "run", f"step-{4000 + int(share * 100) + again}_ckpt"))
                    sv = one_save(tight, cid)
                    for v in sd.values():
                        v.zero_() if v.is_contiguous() else v.fill_(0)
                    gc.collect()
                    torch.cuda.synchronize()
                    t1 = time.perf_counter()
                    dcp.load(sd, checkpoint_id=cid.data, storage_reader=MemoryStorageReader(cid.data, tight_loader), no_dist=True)
                    torch.cuda.synchronize()
                    t2 = time.perf_counter()
                    wrong = [k for k, v in sd.items() if workloads.fingerprint(v) != prints[k]]
                    manager.delete_container(cid)
                    if wrong:
                        break
                tight.release_device_memory()
                limited[f"{room / 1e9:.0f}_GB_of_room"] = {
                    "save_s": round(sv["save"], 3), "blocking_save_ms": round(sv["blocking"] * 1e3, 1),
                    "save_windows": sv["stats"].get("windows", 0), "restore_s": round(t2 - t1, 3),
                    "restore_windows": tight_loader.last_load_stats.get("windows", 0),
                    "restored_bit_identical": not wrong}
                for made in (getattr(tight, "_engine", None), getattr(tight_loader, "_engine", None)):
                    if made is not None:
                        made.destroy()
                del tight, tight_loader
                torch.cuda.empty_cache()

        # ---- a save whose transfer runs on a thread while the device is kept busy, as by a training step ----
        busy = None
        if not args.no_busy_gpu_probe and max_image is None:
            busy = _busy_gpu_probe(device, make_saver(args.save_crc, background_write=True), sd, root, manager)

        # ---- the host link by itself: device <-> the engine's pinned slots, nothing behind them ----
        link = None
        if not args.no_link_probe:
            probe_bytes = min(24 << 30, max(file_bytes, 64 << 20))  # long enough to be past the link's start-up
            # out of the allocator's cache, i.e. the memory the images of the timed steps lay in: a block that the
            # driver has just handed out afresh, while it is still clearing what was released, has measured as low as
            # 46 GB/s in one direction or the other
            scratch = torch.zeros(probe_bytes, dtype=torch.uint8, device=device)
            torch.cuda.synchronize()
            engine = saver._get_engine()
            down, up = [], []
            for _ in range(3):  # directions alternate, the best of each counts
                down.append(engine.link_probe(scratch.data_ptr(), probe_bytes, True))
                up.append(engine.link_probe(scratch.data_ptr(), probe_bytes, False))
            down, up = min(down), min(up)
            del scratch
            link = {"d2h_probe_GBps": round(probe_bytes / 1e9 / down, 2), "h2d_probe_GBps": round(probe_bytes / 1e9 / up, 2),
                    "pcie_gen5_x16_GBps": 64.0,
                    "bytes": probe_bytes, "slot_mib": args.slot_mib, "streams": 2,
                    "what": "probe: pinned hipMemcpyAsync between HBM and the copy engine's own slots, no host-side copy, "
                            "best of three per direction - a measurement of the link on this box in this run, not a "
                            "ceiling (a transfer can come out a little above it); 64 GB/s is the link's nominal rate"}

        # ---- the device's own copy rate, beside which the pack's figure is to be read ----
        copy_probe = None
        if not args.no_link_probe and max_image is None:
            copy_probe = _hbm_copy_probe(device, args.tile_bytes, args.block_threads)

        step_s = mean(rec["step"])
        gb = file_bytes / 1e9
        unpack_s = mean(rec["unpack_ms"]) * 1e-3
        pack_gbps = algorithmic / 1e9 / pack_s if pack_s > 0 else 0.0
        save_gbps, restore_gbps = gb / mean(rec["save"]), gb / mean(rec["restore"])
        if link:
            link["save_frac_of_probe"] = round(save_gbps / link["d2h_probe_GBps"], 4)
            link["restore_frac_of_probe"] = round(restore_gbps / link["h2d_probe_GBps"], 4)
            link["save_frac_of_pcie"] = round(save_gbps / link["pcie_gen5_x16_GBps"], 4)
            link["restore_frac_of_pcie"] = round(restore_gbps / link["pcie_gen5_x16_GBps"], 4)
        # (the host threads' checksums leave the pack what it is without checksums: the flat kernel)
        ratio = PACK_TRAFFIC_RATIO.get((args.workload, "fused" if args.save_crc == "fused" else "beside")) \
            if args.scale >= 1.0 and max_image is None else None
        ms = lambda key: round(mean(rec[key]) * 1e3, 2)  # noqa: E731
        # (an upload that began before the headers were parsed runs beside the parsing and the table: the longer of
        # the two counts)
        beside = mean(rec["r_early"]) > 0
        # (window by window, the checksum pass of one window runs while the next crosses the link)
        restore_known = sum(mean(rec[k]) for k in ("r_unpack_plan", "r_unpack", "r_commit")) + (
            0.0 if mean(rec["r_windows"]) > 1 else mean(rec["r_crc"])) + (
            max(mean(rec["h2d"]), mean(rec["r_parse"]) + mean(rec["r_table"])) if beside else
            mean(rec["h2d"]) + mean(rec["r_parse"]) + mean(rec["r_table"]))
        result = {
            "metric": "save/restore GB/s + blocking save ms, 8B bf16+fp32-Adam shard, 1 MI355X",
            "value": round(2 * gb / step_s, 3),
            "unit": "GB/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(step_s * 1e3, 2),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "u8",
            "data": "synthetic",
            "config": {"workload": f"{args.workload}: {label}", "tensors": len(sd), "payload_bytes": payload,
                       "file_bytes": file_bytes, "scale": args.scale, "tile_bytes": args.tile_bytes or 4096,
                       "engine": {"slot_mib": args.slot_mib, "slots": args.slots, "copy_threads": engine_cfg.resolved_copy_threads()},
                       "crc_chunk_mib": args.crc_chunk_mib, "save_crc": args.save_crc, "restore_crc": args.restore_crc,
                       "plan_cache": args.plan_cache, "save_io": args.save_io, "restore_io": args.restore_io,
                       "max_image_gb": args.max_image_gb, "pool_prefault": not args.no_prefault,
                       "busy_gpu_probe": not args.no_busy_gpu_probe,
                       "restore": "one image" if args.whole_image_restore else "two alternating buffers"},
            **({"partial_restore": partial} if partial else {}),
            "save_GBps": round(save_gbps, 3),
            "restore_GBps": round(restore_gbps, 3),
            "blocking_save_ms": round(mean(rec["blocking"]) * 1e3, 2),
            "blocking_breakdown_ms": {"dcp_plan": ms("plan"), "layout_and_pack_launch": ms("pack_launch"),
                                      "pack_kernel": round(pack_s * 1e3, 3)},
            # host work in the blocking window per tensor: planning + layout + launch, without the kernel itself
            "blocking_host_us_per_tensor": round((mean(rec["blocking"]) - pack_s) * 1e6 / max(len(sd), 1), 2),
            # after the last byte is in the buffer: results, the .metadata file (pickled on a thread of its own while
            # the image crosses the link; see MemoryStorageWriter), finalize
            "save_tail_ms": ms("save_tail"),
            # the first save and restore of the job (iteration 0), not among the timed steps; the pool's file was
            # created `pool_age_s` before it and its pages took `pool_prefault_s` to allocate and map in the background
            "first_save_s": round(first["save"], 3), "first_restore_s": round(first["restore"], 3),
            "first_blocking_save_ms": round(first["blocking"] * 1e3, 2),
            "pool_prefault_s": round(pool_prefault_s, 3), "pool_age_at_first_save_s": round(pool_age_s, 2),
            "restore_breakdown_ms": {
                "dcp_plan_and_metadata": round((mean(rec["restore"]) - mean(rec["r_read"])) * 1e3, 2),
                "parse_headers_resolve_targets": ms("r_parse"), "descriptor_table": ms("r_table"), "h2d": ms("h2d"),
                "h2d_beside_parse_and_table": beside,
                "of_h2d_filling_pinned_slots": ms("h2d_host"),  # pread() into the slots, overlapped with the copies
                "checksum_pass": ms("r_crc"), "checksum_pass_beside_h2d": mean(rec["r_windows"]) > 1,
                "unpack_plan": ms("r_unpack_plan"),
                "unpack_plans_built_beside_h2d": ms("r_plan_beside"), "windows": int(mean(rec["r_windows"])),
                "unpack_and_sync": ms("r_unpack"), "commit": ms("r_commit"),
                "other_in_read_data": round((mean(rec["r_read"]) - restore_known) * 1e3, 2)},
            "pack_GBps": round(pack_gbps, 1),
            # the unpack kernels on an otherwise idle device; in the default restore of a large object they run window by
            # window beside the copies that fill the other buffer (and hide behind them): that sum is the second figure
            "unpack_GBps": round(2 * clean_unpack[1] / 1e9 / clean_unpack[0], 1) if clean_unpack and clean_unpack[0] > 0 else (
                round(2 * mean(rec["unpack_bytes"]) / 1e9 / unpack_s, 1) if unpack_s > 0 else None),
            **({"unpack_GBps_beside_h2d": round(2 * mean(rec["unpack_bytes"]) / 1e9 / unpack_s, 1)} if clean_unpack and unpack_s > 0 else {}),
            "d2h_GBps": round(mean(rec["d2h_bytes"]) / 1e9 / mean(rec["d2h"]), 2) if mean(rec["d2h"]) > 0 else None,
            **({"host_copy_GBps": round(mean(rec["host_copy_bytes"]) / 1e9 / mean(rec["host_copy_s"]), 2),
                "host_copy_bytes": int(mean(rec["host_copy_bytes"]))} if mean(rec["host_copy_s"]) > 0 else {}),
            "h2d_GBps": round(mean(rec["h2d_bytes"]) / 1e9 / mean(rec["h2d"]), 2) if mean(rec["h2d"]) > 0 else None,
            **({"save_windows": int(mean(rec["windows"])), "save_image_pieces": int(mean(rec["image_pieces"]))}
               if mean(rec["windows"]) or mean(rec["image_pieces"]) else {}),
            **({"link_roofline": link} if link else {}),
            **({"hbm_copy_probe": copy_probe} if copy_probe else {}),
            **({"crc_modes": crc_modes} if crc_modes else {}),
            **({"with_dcp_plan_cache": with_cache} if with_cache else {}),
            **({"beside_a_busy_gpu": busy} if busy else {}),
            **({"with_room_for_part_of_the_image": limited} if limited else {}),
            "parity": "restored tensors bit-identical to originals (fingerprints)",
            "roofline": {"bound": "hbm",
                         "kernel": "mlf_fused_crc_kernel<pack> (copy + CRC-32C)" if args.save_crc == "fused" else "mlf_flat_kernel<pack>",
                         "achieved": round(pack_gbps, 1),
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(pack_gbps / HBM_PEAK_GBPS, 4),
                         "traffic": int(ratio * algorithmic) if ratio else None,
                         "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this workload at this scale (profiles/), "
                                           "applied to this run's byte count" if ratio else None,
                         "algorithmic_bytes_per_launch": int(algorithmic),
                         "avg_launch_ms": round(pack_s * 1e3, 3)},
        }
        if args.cpu_baseline_gb > 0:
            result["cpu_baseline"] = cpu_baseline(sd, args.cpu_baseline_gb * 1e9, root, device,
                                                  passes=getattr(args, "cpu_baseline_passes", 5))
    finally:
        try:
            manager.teardown_pool()
        except Exception:
            pass
        mgr.shutdown()
        shutil.rmtree(root, ignore_errors=True)
        # the next workload of this process starts from an empty device
        try:
            saver.release_device_memory()
            loader_engine = getattr(loader, "_engine", None)
            if loader_engine is not None:
                loader_engine.destroy()
                loader._engine = None
        except Exception:
            pass
        sd.clear()
        del parents
        gc.collect()
        torch.cuda.empty_cache()
    return result


if __name__ == "__main__":
    main()
