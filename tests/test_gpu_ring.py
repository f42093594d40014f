"""The ring all-reduce drop-in (tirocinio-triennale_amd/host/allreduce_ring.hpp) with its ranks as
host threads on one GPU, checked against the CPU oracle: every rank must end with the bytes that
the reference's schedule (HomComp/src/cuda_awareallreduce.cu:166-265, :436-585) gives, i.e. block
b compressed by rank b, summed homomorphically by ranks b+1 ... b+R-1 in that order, decompressed."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "ring_allreduce")


def blocks_equal(count, ranks):
    """HomComp/src/cuda_awareallreduce.cu:189-190."""
    block = (count + ranks - 1) // ranks
    block = (block + 32767) // 32768 * 32768
    return [b * block for b in range(ranks)], [block] * ranks, block * ranks


def blocks_seg(count, ranks):
    """HomComp/src/cuda_awareallreduce.cu:455-489."""
    pad = (count + 32767) // 32768 * 32768
    early = late = pad // ranks
    split = pad % ranks
    if split:
        early += 1
    early += (-early) % 4
    late += (-late) % 4
    offs, cnts = [], []
    for b in range(ranks):
        off = b * early if b < split else split * early + (b - split) * late
        cnt = early if b < split else late
        if b == ranks - 1:
            cnt = max(count - off, 0)   # the reference's count goes negative here; the drop-in's block is empty
        offs.append(off)
        cnts.append(cnt)
    return offs, cnts, max(early * split + late * (ranks - split), count)


def expected(orc, data, count, eb, variant):
    ranks = len(data)
    offs, cnts, padded = (blocks_seg if "seg" in variant else blocks_equal)(count, ranks)
    full = [np.concatenate([d, np.zeros(padded - count, np.float32)]) for d in data]
    out = np.zeros(padded, np.float32)
    for b in range(ranks):
        if cnts[b] == 0:
            continue
        sl = slice(offs[b], offs[b] + cnts[b])
        stream = orc.compress(full[b][sl], eb)
        for k in range(1, ranks):
            local = full[(b + k) % ranks][sl]
            if variant.startswith("I"):
                stream = orc.hom_sum_i32(stream, orc.quant_predict(local, eb))
            else:
                stream = orc.hom_sum_f32(stream, local, eb)
        out[sl] = orc.decompress(stream, cnts[b], eb)
    return out[:count]


@pytest.mark.parametrize("variant,ranks,count", [
    ("F", 4, 4 * 32768 * 3),           # the reference's own domain: blocks that are multiples of 32768
    ("F", 8, 1_000_003),               # padded blocks, a last block that is mostly padding
    ("I", 4, 500_000),                 # Lorenzo pre-pass + integer homomorphic sum
    ("Fseg", 8, 1_000_003),            # uneven blocks, last block ends with the array
    ("Iseg", 3, 700_001),
    ("Fseg", 8, 100_000),              # padding pushes the last block's start beyond the array: an empty block
    ("Fopt", 2, 262_144),              # two ranks: no intermediate step
])
def test_ring_allreduce(tmp_path, orc, gen, cuda, variant, ranks, count):
    assert os.path.exists(EXE), "tests/cpp/ring_allreduce is not built (run __graft_entry__.build())"
    orc.set_threads(16)
    check_ring_allreduce(EXE, tmp_path, orc, gen, variant, ranks, count, timeout=100)


def check_ring_allreduce(exe, tmp_path, orc, gen, variant, ranks, count, timeout):
    """Runs the program `exe` (the drop-in on the GPU, or its host build on the CPU execution model)
    and compares every rank's result with the oracle's."""
    data = [gen.smooth_np(count, 70 + r) for r in range(ranks)]
    mn, mx = orc.value_range(np.concatenate(data))
    eb = orc.rel_to_abs(1e-4, mn, mx)
    inp, outp = tmp_path / "in", tmp_path / "out"
    for r, d in enumerate(data):
        d.tofile(f"{inp}.r{r}.f32")
    res = subprocess.run([exe, variant, str(ranks), str(count), repr(float(eb)), str(inp), str(outp), "2"],
                         capture_output=True, text=True, timeout=timeout)
    assert res.returncode == 0 and "status=0" in res.stdout, res.stdout + res.stderr
    want = expected(orc, data, count, eb, variant)
    for r in range(ranks):
        got = np.fromfile(f"{outp}.r{r}.f32", np.float32)
        assert got.size == count
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"rank {r}"
    # the error of the reduced values stays within ranks * eb (plus float32 rounding of the reference sum)
    exact = np.zeros(count, np.float64)
    for d in data:
        exact += d
    assert (np.abs(want.astype(np.float64) - exact) <= ranks * float(eb) * (1 + 1e-3)).all()
