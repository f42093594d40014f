"""Host logic of the ring all-reduce drop-in: the block layouts of
tirocinio-triennale_amd/host/allreduce_ring.hpp against the reference's rules
(HomComp/src/cuda_awareallreduce.cu:189-190 equal blocks; :455-489 segmented blocks), restated here
from the reference text, and against what any layout must satisfy.  Runs without a GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "ring_blocks")


def layout(kind, count, ranks):
    if not os.path.exists(EXE):   # normally built by __graft_entry__.build(); a host-only program
        subprocess.run(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O2", "-std=c++17", "-o", EXE, EXE + ".cpp"],
                       check=True, timeout=300)
    out = subprocess.run([EXE, kind, str(count), str(ranks)], capture_output=True, text=True, timeout=30, check=True)
    rows = [tuple(int(v) for v in line.split()) for line in out.stdout.split("\n") if line]
    return rows[:-1], rows[-1]


@pytest.mark.parametrize("count", [1, 32768, 100_000, 1_000_003, 3 * 32768 * 8, (1 << 25) + 5])
@pytest.mark.parametrize("ranks", [2, 3, 4, 8])
def test_equal_blocks(count, ranks):
    blocks, (padded, max_count) = layout("equal", count, ranks)
    block = -(-count // ranks)
    block = -(-block // 32768) * 32768          # :189-190
    assert blocks == [(b * block, block) for b in range(ranks)]
    assert padded == block * ranks >= count and max_count == block


@pytest.mark.parametrize("count", [1, 32768, 100_000, 1_000_003, 3 * 32768 * 8, (1 << 25) + 5])
@pytest.mark.parametrize("ranks", [2, 3, 4, 8])
def test_segmented_blocks(count, ranks):
    blocks, (padded, max_count) = layout("seg", count, ranks)
    pad = -(-count // 32768) * 32768
    late = pad // ranks                           # COLL_BASE_COMPUTE_BLOCKCOUNT
    split = pad % ranks
    early = late + 1 if split else late
    early += (-early) % 4                         # :460-465
    late += (-late) % 4
    off = 0
    for b, (o, c) in enumerate(blocks):
        assert o == off and o % 4 == 0
        want = early if b < split else late
        if b == ranks - 1:
            # :486-487: the last block ends with the array.  Where the padding pushes its start
            # beyond the array the reference's count goes negative; here the block is empty.
            want = max(count - o, 0)
        assert c == want
        off += early if b < split else late
    if count >= blocks[-1][0]:
        assert sum(c for _, c in blocks) == count
    # the blocks are disjoint, in order, and cover the array
    assert all(blocks[b][0] + blocks[b][1] <= blocks[b + 1][0] for b in range(ranks - 1))
    assert max(o + c for o, c in blocks) >= count
    assert max_count == early and padded >= count
    assert padded >= max(o + c for o, c in blocks)
