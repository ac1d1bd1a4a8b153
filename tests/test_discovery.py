"""Recovery discovery (host logic, CPU only).  The expectations restate those of the reference's own tests
(tests/core/test_checkpoint_loader.py:763-1320 plan/selection, :1332-1700 candidates, :1717-1800 retrieval,
:426-540 fetch on read), driven through injected collectives instead of mocks of torch.distributed."""

import os
import pickle

import numpy as np
import pytest
from torch.distributed.checkpoint.filesystem import _StorageInfo
from torch.distributed.checkpoint.metadata import Metadata

from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core import checkpoint_discovery
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader


class _Cluster:
    """Collectives of a job whose other ranks' contributions are scripted by the test."""

    def __init__(self, rank=0, world=1, others=None):
        self.rank, self.world = rank, world
        self.others = others or {}  # call number -> {rank: contribution}
        self.gathers, self.broadcasts = [], []

    def all_gather(self, out_list, obj):
        scripted = self.others.get(len(self.gathers), {})
        for r in range(self.world):
            out_list[r] = obj if r == self.rank else scripted.get(r)
        self.gathers.append(obj)

    def broadcast(self, obj_list, src=0):
        self.broadcasts.append((list(obj_list), src))


class _Replication:
    def __init__(self, ok=True, create=False):
        self.ok, self.create, self.calls = ok, create, []

    def sync_bulk_retrieve(self, source_global_rank, object_ids_to_retrieve, container_ids_to_retrieve):
        self.calls.append((source_global_rank, [o.data for o in object_ids_to_retrieve]))
        if self.ok and self.create:
            for o in object_ids_to_retrieve:
                os.makedirs(os.path.dirname(o.data), exist_ok=True)
                open(o.data, "wb").write(b"fetched")
        return self.ok


def _loader(cluster=None, replication=None, nodes=1, monkeypatch=None, **kw):
    cluster = cluster or _Cluster()
    if monkeypatch is not None:
        monkeypatch.setattr(checkpoint_discovery, "get_num_of_nodes", lambda: nodes)
    return DefaultMLFlashpointCheckpointLoader(
        CheckpointObjectManager(), replication, global_rank_getter=lambda: cluster.rank, local_rank_getter=lambda: 0,
        broadcast_object_list_func=cluster.broadcast, all_gather_object_func=cluster.all_gather,
        world_size_getter=lambda: cluster.world, **kw)


def _metadata(paths):
    md = Metadata(state_dict_metadata={})
    md.storage_data = {i: _StorageInfo(relative_path=p, offset=0, length=100) for i, p in enumerate(paths)}
    return md


def _make_checkpoint(base, step, objects=("__0_0_src0.distcp",), common=True, metadata=True):
    d = os.path.join(base, f"step-{step}_ckpt")
    os.makedirs(d)
    for name in objects:
        open(os.path.join(d, name), "wb").write(b"x" * 10)
    if common:
        open(os.path.join(d, "common.pt"), "wb").write(b"c")
    if metadata:
        with open(os.path.join(d, ".metadata"), "wb") as f:
            pickle.dump(_metadata(list(objects)), f)
    return d


# ---- candidates ----------------------------------------------------------------------------------------------
def test_candidates_single_node_sorted_numerically_and_skip_unfinished(tmp_path):
    base = CheckpointContainerId(str(tmp_path))
    loader = _loader()
    assert loader.get_candidate_checkpoints(CheckpointContainerId(str(tmp_path / "absent"))) == []
    for step in (9, 10, 100, 2):
        (tmp_path / f"step-{step}_ckpt").mkdir()
    (tmp_path / "other_dir").mkdir()
    (tmp_path / "step-100_ckpt__0__unfinished").touch()
    got = loader.get_candidate_checkpoints(base)
    assert [os.path.basename(c.data) for c in got] == ["step-10_ckpt", "step-9_ckpt", "step-2_ckpt"]


def test_candidates_are_the_intersection_of_the_non_empty_lists(tmp_path):
    base = CheckpointContainerId(str(tmp_path))
    (tmp_path / "step-100_ckpt").mkdir()
    (tmp_path / "step-200_ckpt").mkdir()
    p = lambda s: str(tmp_path / f"step-{s}_ckpt")  # noqa: E731
    # the other node has nothing at all: its empty list does not veto
    got = _loader(_Cluster(world=2, others={0: {1: []}})).get_candidate_checkpoints(base)
    assert [c.data for c in got] == [p(200), p(100)]
    # the other node has {200, 300}: only 200 is common
    got = _loader(_Cluster(world=2, others={0: {1: [p(200), p(300)]}})).get_candidate_checkpoints(base)
    assert [c.data for c in got] == [p(200)]
    # disjoint
    assert _loader(_Cluster(world=2, others={0: {1: [p(300)]}})).get_candidate_checkpoints(base) == []
    # a non-zero rank sees the same answer and no broadcast is involved
    cluster = _Cluster(rank=1, world=2, others={0: {0: [p(200), p(100)]}})
    got = _loader(cluster).get_candidate_checkpoints(base)
    assert [c.data for c in got] == [p(200), p(100)] and cluster.broadcasts == []


# ---- objects by rank -------------------------------------------------------------------------------------------
def test_objects_by_rank_lists_local_entries_and_fills_the_location_cache(tmp_path):
    d = _make_checkpoint(str(tmp_path), 7, objects=("a_src0.distcp", "b_src0.distcp"))
    cid = CheckpointContainerId(d)
    remote = [CheckpointObjectId(os.path.join(d, "c_src1.distcp")), CheckpointObjectId(os.path.join(d, ".metadata"))]
    loader = _loader(_Cluster(world=3, others={0: {1: remote, 2: None}}))
    by_rank = loader.get_checkpoint_objects_by_rank(cid)
    assert sorted(os.path.basename(o.data) for o in by_rank[0]) == [".metadata", "a_src0.distcp", "b_src0.distcp", "common.pt"]
    assert by_rank[1] == remote and by_rank[2] == []
    cache = loader._available_objects_cache[cid]
    assert cache[os.path.join(d, ".metadata")] == [0, 1] and cache[os.path.join(d, "c_src1.distcp")] == [1]
    # a container that is not a directory contributes nothing
    assert _loader().get_checkpoint_objects_by_rank(CheckpointContainerId(str(tmp_path / "nope"))) == {0: []}


# ---- retrieval plan ----------------------------------------------------------------------------------------------
def test_retrieval_plan_known_answers(monkeypatch):
    ckpt = CheckpointContainerId("/tmp/ckpt")
    loader = _loader(_Cluster(world=2), nodes=2, monkeypatch=monkeypatch)
    oid = lambda *names: [CheckpointObjectId(f"/tmp/ckpt/{n}") for n in names]  # noqa: E731
    monkeypatch.setattr(loader, "read_metadata", lambda c: _metadata(["src0/obj", "src1/obj"]))
    # each rank holds the other's object; rank 0 also has the per-node files, rank 1 (first of node 2) does not
    plan = loader._compute_retrieval_plan(ckpt, {0: oid("src1/obj", "common.pt", ".metadata"), 1: oid("src0/obj")})
    assert plan[0] == [(1, "/tmp/ckpt/src0/obj")]
    assert sorted(plan[1]) == [(0, "/tmp/ckpt/.metadata"), (0, "/tmp/ckpt/common.pt"), (0, "/tmp/ckpt/src1/obj")]
    # an object nobody has: not viable
    assert loader._compute_retrieval_plan(ckpt, {0: [], 1: []}) is None
    # no storage data, or unreadable metadata: not viable
    md = _metadata([])
    md.storage_data = None
    monkeypatch.setattr(loader, "read_metadata", lambda c: md)
    assert loader._compute_retrieval_plan(ckpt, {0: []}) is None

    def boom(c):
        raise OSError("unreadable")

    monkeypatch.setattr(loader, "read_metadata", boom)
    assert loader._compute_retrieval_plan(ckpt, {0: []}) is None


def test_one_node_two_ranks_sharing_storage_need_nothing(monkeypatch):
    ckpt = CheckpointContainerId("/tmp/checkpoints/step-100_ckpt")
    loader = _loader(_Cluster(world=2), nodes=1, monkeypatch=monkeypatch)
    monkeypatch.setattr(loader, "read_metadata", lambda c: _metadata(["/src0/obj", "/src1/obj"]))
    common = [CheckpointObjectId(f"{ckpt.data}/.metadata"), CheckpointObjectId(f"{ckpt.data}/common.pt")]
    plan = loader._compute_retrieval_plan(ckpt, {0: [CheckpointObjectId(f"{ckpt.data}/src0/obj")] + common,
                                                1: [CheckpointObjectId(f"{ckpt.data}/src1/obj")] + common})
    assert not plan.get(0) and not plan.get(1)


# ---- selection -------------------------------------------------------------------------------------------------------
def test_latest_complete_checkpoint_single_process(tmp_path):
    base = CheckpointContainerId(str(tmp_path / "job"))
    loader = _loader()
    assert loader.get_latest_complete_checkpoint(base) is None
    _make_checkpoint(base.data, 5)
    _make_checkpoint(base.data, 10)
    _make_checkpoint(base.data, 20, metadata=False)            # no .metadata: skipped
    _make_checkpoint(base.data, 30, objects=())                # metadata names nothing, still complete
    _make_checkpoint(base.data, 40)
    os.remove(os.path.join(base.data, "step-40_ckpt", "__0_0_src0.distcp"))  # needed object missing everywhere
    _make_checkpoint(base.data, 50)
    open(os.path.join(base.data, "step-50_ckpt__0__unfinished"), "w").close()  # still being written
    assert loader.get_latest_complete_checkpoint(base).data == os.path.join(base.data, "step-30_ckpt")
    os.remove(os.path.join(base.data, "step-50_ckpt__0__unfinished"))
    assert loader.get_latest_complete_checkpoint(base).data == os.path.join(base.data, "step-50_ckpt")


def test_common_state_requirement_follows_the_reference_and_can_be_dropped(tmp_path):
    base = CheckpointContainerId(str(tmp_path / "job"))
    _make_checkpoint(base.data, 1, common=False)  # what plain dcp.save leaves behind
    loader = _loader()
    assert loader.get_latest_complete_checkpoint(base) is None
    loader.common_state_object_name = None
    assert loader.get_latest_complete_checkpoint(base).data.endswith("step-1_ckpt")


def test_planner_is_the_lowest_rank_with_metadata_and_its_plan_is_broadcast(tmp_path, monkeypatch):
    base = CheckpointContainerId(str(tmp_path / "job"))
    d = _make_checkpoint(base.data, 100, objects=("x_src0.distcp",))
    # rank 1 (second node) has only the data object of rank 1: it must fetch .metadata and common.pt from rank 0
    there = [CheckpointObjectId(os.path.join(d, "y_src1.distcp"))]
    cluster = _Cluster(world=2, others={0: {1: [d]}, 1: {1: there}, 2: {1: True}})
    repl = _Replication(ok=True)
    loader = _loader(cluster, repl, nodes=2, monkeypatch=monkeypatch)
    monkeypatch.setattr(loader, "read_metadata", lambda c: _metadata(["x_src0.distcp", "y_src1.distcp"]))
    assert loader.get_latest_complete_checkpoint(base).data == d
    (sent, src), = cluster.broadcasts
    assert src == 0 and sorted(sent[0][1]) == [(0, os.path.join(d, ".metadata")), (0, os.path.join(d, "common.pt"))]
    assert 0 not in sent[0] and repl.calls == []  # rank 0 itself had nothing to fetch


def test_failed_retrieval_moves_on_to_the_next_candidate(tmp_path, monkeypatch):
    base = CheckpointContainerId(str(tmp_path / "job"))
    old = _make_checkpoint(base.data, 1)
    new = _make_checkpoint(base.data, 2)
    os.remove(os.path.join(new, "__0_0_src0.distcp"))  # this rank lost its object; rank 1 still has a replica
    replica = [CheckpointObjectId(os.path.join(new, "__0_0_src0.distcp"))]
    script = {0: {1: [old, new]}, 1: {1: replica}, 2: {1: True}, 3: {1: []}}
    repl = _Replication(ok=False)
    loader = _loader(_Cluster(world=2, others=script), repl, nodes=1, monkeypatch=monkeypatch)
    assert loader.get_latest_complete_checkpoint(base).data == old
    assert repl.calls == [(1, [os.path.join(new, "__0_0_src0.distcp")])]
    # with a working replication layer the newer checkpoint is recovered
    repl = _Replication(ok=True, create=True)
    loader = _loader(_Cluster(world=2, others=script), repl, nodes=1, monkeypatch=monkeypatch)
    assert loader.get_latest_complete_checkpoint(base).data == new
    assert open(os.path.join(new, "__0_0_src0.distcp"), "rb").read() == b"fetched"


def test_retrieve_checkpoint_outcome_is_agreed_across_ranks():
    plan = {0: [(1, "/c/a"), (1, "/c/b"), (2, "/c/c")]}
    repl = _Replication(ok=True)
    loader = _loader(_Cluster(world=3, others={0: {1: True, 2: True}}), repl)
    assert loader.retrieve_checkpoint(plan) is True
    assert repl.calls == [(1, ["/c/a", "/c/b"]), (2, ["/c/c"])]  # grouped by source rank
    loader = _loader(_Cluster(world=3, others={0: {1: True, 2: False}}), _Replication(ok=True))
    assert loader.retrieve_checkpoint(plan) is False              # another rank failed
    loader = _loader(_Cluster(rank=1, world=3, others={0: {0: True, 2: True}}), repl)
    assert loader.retrieve_checkpoint(plan) is True and len(repl.calls) == 2  # nothing to fetch on rank 1


# ---- fetch on read ---------------------------------------------------------------------------------------------------
def test_missing_object_is_fetched_on_read_from_a_rank_that_listed_it(tmp_path):
    ckpt = CheckpointContainerId(str(tmp_path / "step-1_ckpt"))
    os.makedirs(ckpt.data)
    oid = CheckpointObjectId.from_container(ckpt, "data_src0.distcp")
    loader = _loader()
    with pytest.raises(FileNotFoundError, match="does not exist on any node in the cluster"):
        loader.read_data(oid, [], None, {})                      # no replication manager at all
    loader = _loader(replication=_Replication(ok=True, create=True))
    with pytest.raises(FileNotFoundError):
        loader.read_data(oid, [], None, {})                      # nobody listed the object
    loader._available_objects_cache[ckpt] = {oid.data: [3, 5]}
    assert loader._try_retrieve_object_if_missing(oid) is True
    assert loader._replication_manager.calls == [(3, [oid.data])] and os.path.exists(oid.data)
    assert loader._try_retrieve_object_if_missing(oid) is True and len(loader._replication_manager.calls) == 1
    os.remove(oid.data)
    loader._replication_manager = _Replication(ok=False)
    assert loader._try_retrieve_object_if_missing(oid) is False


# ---- checksum verification while choosing ------------------------------------------------------------------------------
def test_corrupted_object_counts_as_missing_when_verification_is_on(tmp_path):
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    base = CheckpointContainerId(str(tmp_path / "job"))
    chunk = 1 << 16
    payload = np.random.default_rng(3).integers(0, 256, 5 * chunk + 123, dtype=np.uint8)
    for step in (1, 2):
        d = _make_checkpoint(base.data, step)
        obj = os.path.join(d, "__0_0_src0.distcp")
        open(obj, "wb").write(bytes(METADATA_SIZE) + payload.tobytes())
        crcs = [P.crc32c_host(payload.ctypes.data + o, min(chunk, len(payload) - o)) for o in range(0, len(payload), chunk)]
        integrity.write_sidecar(obj, chunk, len(payload), np.array(crcs, dtype=np.uint32))
    bad = os.path.join(base.data, "step-2_ckpt", "__0_0_src0.distcp")
    with open(bad, "r+b") as f:  # one flipped bit in the fourth chunk
        f.seek(METADATA_SIZE + 3 * chunk + 77)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 1]))
    assert _loader().get_latest_complete_checkpoint(base).data.endswith("step-2_ckpt")  # presence only, as the reference
    checking = _loader(verify_on_discovery=True)
    assert checking._object_is_intact(bad) is False
    assert checking._object_is_intact(os.path.join(base.data, "step-1_ckpt", "__0_0_src0.distcp")) is True
    assert checking.get_latest_complete_checkpoint(base).data.endswith("step-1_ckpt")
    with open(bad, "ab") as f:  # a truncated or extended object fails the check as well
        f.write(b"tail")
    assert checking._object_is_intact(bad) is False
