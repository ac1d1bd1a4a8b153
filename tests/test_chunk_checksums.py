"""Per-chunk checksums joined from the checksums of pieces (``hip/integrity.py: ChunkChecksums``), against the
oracle's CRC-32C of the chunks themselves.  Host logic only."""

import numpy as np
import pytest

from ml_flashpoint.hip import integrity


def _chunks_of(oracle_c, data: bytes, chunk: int) -> list:
    return [oracle_c.oracle_crc32c(data[o : o + chunk], len(data[o : o + chunk])) for o in range(0, len(data), chunk)]


@pytest.mark.parametrize("chunk", [64, 100, 4096])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_pieces_cut_anywhere_give_the_chunks_of_the_whole(oracle_c, chunk, seed):
    rng = np.random.default_rng(seed)
    total = int(rng.integers(1, 9 * chunk))
    data = rng.integers(0, 256, total, dtype=np.uint8).tobytes()
    # pieces end anywhere: inside a chunk, on a boundary, several per chunk, several chunks per piece
    ends = sorted(set(rng.integers(1, total + 1, int(rng.integers(1, 12))).tolist()) | {total})
    sums = integrity.ChunkChecksums(chunk, total)
    at = 0
    for end in ends:
        parts = integrity.ChunkChecksums.cuts(at, end - at, chunk)
        assert parts[0][0] == at and sum(n for _, n in parts) == end - at
        assert all((first + n) % chunk == 0 for first, n in parts[:-1])  # every part but the last ends on a boundary
        sums.add(at, end - at, [oracle_c.oracle_crc32c(data[first : first + n], n) for first, n in parts])
        at = end
    assert sums.result().tolist() == _chunks_of(oracle_c, data, chunk)


def test_gaps_wrong_counts_and_incomplete_sections_are_refused(oracle_c):
    sums = integrity.ChunkChecksums(64, 200)
    sums.add(0, 70, [1, 2])
    with pytest.raises(ValueError, match="does not continue"):
        sums.add(80, 10, [3])
    with pytest.raises(ValueError, match="checksums for"):
        sums.add(70, 100, [3])
    with pytest.raises(ValueError, match="cover 70 of 200"):
        sums.result()
    assert integrity.ChunkChecksums(64, 0).result().tolist() == []
    with pytest.raises(ValueError):
        integrity.ChunkChecksums(0, 10)


def test_the_library_and_the_oracle_agree_on_the_law_that_joins_them(oracle_c):
    from ml_flashpoint.hip import plan as P

    rng = np.random.default_rng(7)
    for _ in range(50):
        a, b, n = int(rng.integers(0, 1 << 32)), int(rng.integers(0, 1 << 32)), int(rng.integers(0, 1 << 20))  # the oracle shifts bit by bit
        assert P.crc32c_combine(a, b, n) == oracle_c.oracle_crc32c_combine(a, b, n)
