"""The kernels' source text executed on the CPU (tests/emu: lanes as fibers of their wave's thread, workgroups as
processes, device memory as guarded shared mappings) against the oracle, byte for byte, on small
inputs.  It covers what a GPU run covers less directly: every path of every kernel kind on data
that does and does not suit it, whatever the launch heuristics would pick; grids of one and of
many rounds; every LDS budget and deferral depth, spills included; stated sizes that cut a stream
short; and, through the guard pages and the checked buffer descriptors, that no access leaves
its buffer.  It does not cover the compiler, timing or the memory model of the hardware: parity
on the GPU stays with the gpu-marked tests.
"""
import os
import subprocess

import numpy as np
import pytest



@pytest.fixture(scope="module")
def emu(emu_sources, tmp_path_factory):
    return Emu(emu_sources.build(), str(tmp_path_factory.mktemp("emu")))


class Emu:
    # LDS bytes per data wave that the library's launches use, smallest to largest, and one below them
    BUDGETS = (2 * (1024 + 64), 2 * (2048 + 64), 2 * (3072 + 64), 2 * (4992 + 64), 2 * (8192 + 64))

    def __init__(self, binary, tmp):
        self.binary, self.tmp, self.calls = binary, tmp, 0

    def run(self, op, n, eb, a, b=None, groups=2, budget=BUDGETS[2], kind=0, slots=2, plain=0, dtype=np.uint8, offsets=False,
            stated_a=None, env=None, expect=0):
        self.calls += 1
        pa, pb, po, pf = (os.path.join(self.tmp, x) for x in ("a", "b", "out", "ofs"))
        for path, data in ((pa, a), (pb, b)):
            if data is not None:
                np.ascontiguousarray(data).tofile(path)
        args = [self.binary, op, str(n), repr(float(eb)), str(groups), str(budget), str(kind), str(slots), str(plain),
                pa if a is not None else "-", pb if b is not None else "-", po, pf if offsets else "-"]
        if stated_a is not None:
            args.append(str(stated_a))
        r = subprocess.run(args, capture_output=True, text=True, timeout=600, env=dict(os.environ, **(env or {})))
        assert r.returncode == expect, f"{' '.join(args[1:9])}: exit {r.returncode}\n{r.stderr[-3000:]}"
        if expect:
            return r.stderr
        out = np.fromfile(po, dtype=dtype)
        return (out, np.fromfile(pf, dtype=np.uint64)) if offsets else out


def same(got, want, what):
    assert got.size == want.size, f"{what}: {got.size} bytes, oracle {want.size}"
    ne = np.nonzero(got != want)[0]
    assert ne.size == 0, f"{what}: {ne.size} of {got.size} differ, first at {ne[0]}"


def same_f32(got, want, what):
    same(got.view(np.uint32), np.ascontiguousarray(want).view(np.uint32), what)


def bound_of(orc, rel, *arrays):
    lo = min(float(orc.value_range(a)[0]) for a in arrays)
    hi = max(float(orc.value_range(a)[1]) for a in arrays)
    return orc.rel_to_abs(rel, lo, hi)


def operands(gen, orc, name, n):
    """(x, y, eb, few) -- few: the data suits the bit-plane paths for few planes."""
    if name == "smooth_coarse":      # blocks of one to three planes
        x, y = gen.smooth_np(n, seed=1), gen.smooth_np(n, seed=2)
        return x, y, bound_of(orc, 1e-3, x, y), True
    if name == "smooth_fine":        # around eight planes, mostly outlier mode
        x, y = gen.smooth_np(n, seed=1), gen.smooth_np(n, seed=2)
        return x, y, bound_of(orc, 1e-6, x, y), False
    if name == "uniform":
        x, y = gen.uniform_np(n, seed=1), gen.uniform_np(n, seed=2)
        return x, y, bound_of(orc, 1e-2, x, y), False
    if name == "gradient_abs":       # up to 22 planes
        x, y = gen.gradient_like_np(n, seed=1), gen.gradient_like_np(n, seed=2)
        return x, y, np.float32(1e-6), False
    if name == "patchy":             # zero blocks, constant runs, a few spikes, smooth stretches: every block mode within a tile
        x, y = gen.smooth_np(n, seed=5), gen.smooth_np(n, seed=6)
        i = np.arange(n)
        x[(i // 96) % 3 == 0] = 0.0
        y[(i // 160) % 2 == 0] = 0.0
        x[(i // 1000) % 4 == 1] = 0.25
        x[i % 977 == 5] = 3.0
        y[i % 1201 == 7] = -2.0
        return x, y, bound_of(orc, 1e-4, x, y), False
    if name == "any_bits":           # every float32 bit pattern, NaN and infinities included; the conversions saturate
        rng = np.random.default_rng(11)
        x = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32)
        y = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32)
        return x, y, np.float32(1e-3), False
    raise KeyError(name)


def run_all_ops(emu, orc, x, y, eb, n, groups, budget, slots, what):
    """Every stream kernel of every kind on one pair of operands; returns the streams of x and of the sum."""
    ca, cb = orc.compress(x, eb), orc.compress(y, eb)
    want_sum = orc.hom_sum_f32(ca, y, eb)
    cfg = dict(groups=groups, budget=budget, slots=slots)
    same(emu.run("compress", n, eb, x, **cfg), ca, f"{what} compress")
    same_f32(emu.run("decompress", n, eb, ca, dtype=np.float32, **cfg), orc.decompress(ca, n, eb), f"{what} decompress")
    deltas = orc.quant_predict(y, eb)
    want_i32 = orc.hom_sum_i32(ca, deltas)
    for kind in (0, 1):
        same(emu.run("hom_sum_f32", n, eb, ca, y, kind=kind, **cfg), want_sum, f"{what} hom_sum_f32 kind {kind}")
        same(emu.run("hom_sum_i32", n, eb, ca, deltas, kind=kind, **cfg), want_i32, f"{what} hom_sum_i32 kind {kind}")
    want_add = orc.hom_add(ca, cb, n)
    for kind in (1, 2):
        same(emu.run("hom_add", n, eb, ca, cb, kind=kind, **cfg), want_add, f"{what} hom_add kind {kind}")
    return ca, cb, want_sum


DATA = ("smooth_coarse", "smooth_fine", "uniform", "gradient_abs", "patchy", "any_bits")


@pytest.mark.parametrize("name", DATA)
def test_every_kernel_kind_on_every_kind_of_data(emu, orc, gen, name):
    """Three chunks with a ragged end, a grid of several rounds, the middle LDS budget."""
    n = 2 * 32768 + 4097 + 13
    x, y, eb, _ = operands(gen, orc, name, n)
    run_all_ops(emu, orc, x, y, eb, n, groups=2, budget=Emu.BUDGETS[3], slots=2, what=name)


@pytest.mark.parametrize("n", [1, 32, 33, 4095, 4097, 32769])
def test_lengths_around_block_tile_and_chunk(emu, orc, gen, n):
    x, y, eb, _ = operands(gen, orc, "smooth_coarse", 40000)
    run_all_ops(emu, orc, x[:n].copy(), y[:n].copy(), eb, n, groups=1, budget=Emu.BUDGETS[2], slots=2, what=f"n={n}")


@pytest.mark.parametrize("budget,slots", [(Emu.BUDGETS[0], 2), (Emu.BUDGETS[1], 3), (Emu.BUDGETS[2], 4), (Emu.BUDGETS[4], 2)])
@pytest.mark.parametrize("name", ["smooth_coarse", "gradient_abs"])
def test_lds_budgets_and_deferral_depths(emu, orc, gen, name, budget, slots):
    """From slots that hold no tile of the data (everything spills) to slots that hold every tile."""
    n = 32768 + 9000
    x, y, eb, _ = operands(gen, orc, name, n)
    run_all_ops(emu, orc, x, y, eb, n, groups=1, budget=budget, slots=slots, what=f"{name} {budget}/{slots}")


@pytest.mark.parametrize("groups", [1, 3, 5])
def test_grid_shapes(emu, orc, gen, groups):
    """Many rounds per wave, a grid that does not divide the tiles, one tile per wave (20 tiles on 5 x 4 waves)."""
    n = 2 * 32768 + 12345
    x, y, eb, _ = operands(gen, orc, "patchy", n)
    run_all_ops(emu, orc, x, y, eb, n, groups=groups, budget=Emu.BUDGETS[2], slots=3, what=f"groups={groups}")


def test_plain_codec(emu, orc, gen):
    n = 32768 + 555
    for name in ("smooth_coarse", "gradient_abs"):
        x, _, eb, _ = operands(gen, orc, name, n)
        want = orc.compress_plain(x, eb)
        same(emu.run("compress", n, eb, x, plain=1, budget=Emu.BUDGETS[3]), want, f"{name} compress_plain")
        same_f32(emu.run("decompress", n, eb, want, dtype=np.float32), orc.decompress_plain(want, n, eb), f"{name} decompress_plain")


def test_tile_offsets_left_by_a_producing_call(emu, orc, gen):
    n = 32768 + 4096 * 3 + 100
    x, _, eb, _ = operands(gen, orc, "smooth_fine", n)
    want, block_ofs = orc.compress(x, eb, want_offsets=True)
    got, tile_ofs = emu.run("compress", n, eb, x, groups=3, offsets=True)
    same(got, want, "compress")
    assert np.array_equal(tile_ofs, block_ofs[:-1:128]), "tile offsets"


@pytest.mark.parametrize("name", ["smooth_coarse", "smooth_fine"])
def test_stated_size_cuts_the_stream_short(emu, orc, gen, name):
    """Blocks that start at or beyond the stated size count as empty, blocks that start below it are
    read in full (HomComp/src/GSZ.cu:908-911): stated sizes from the header bytes alone to one byte short."""
    n = 32768 + 8192 + 77
    x, y, eb, _ = operands(gen, orc, name, n)
    ca, cb = orc.compress(x, eb), orc.compress(y, eb)
    hdr = orc.header_bytes(n)
    deltas = orc.quant_predict(y, eb)
    for cut in (hdr, hdr + 1, hdr + (ca.size - hdr) // 3, ca.size - 1):
        what = f"{name} stated {cut} of {ca.size}"
        same_f32(emu.run("decompress", n, eb, ca, dtype=np.float32, stated_a=cut), orc.decompress(ca, n, eb, cmp_size=cut),
                 f"{what} decompress")
        for kind in (0, 1):
            same(emu.run("hom_sum_f32", n, eb, ca, y, kind=kind, stated_a=cut), orc.hom_sum_f32(ca, y, eb, cmp_in_size=cut),
                 f"{what} hom_sum_f32 kind {kind}")
            same(emu.run("hom_sum_i32", n, eb, ca, deltas, kind=kind, stated_a=cut), orc.hom_sum_i32(ca, deltas, cmp_in_size=cut),
                 f"{what} hom_sum_i32 kind {kind}")
        for kind in (1, 2):
            same(emu.run("hom_add", n, eb, ca, cb, kind=kind, stated_a=cut), orc.hom_add(ca, cb, n, size_a=cut),
                 f"{what} hom_add kind {kind}")


@pytest.mark.parametrize("n", [4099, 32768 + 4096 * 5 + 21])
@pytest.mark.parametrize("name", ["smooth_coarse", "smooth_fine", "any_bits"])
def test_stated_size_is_the_buffers_capacity(emu, orc, gen, name, n):
    """The ring with its lengths on the device states every incoming stream's size as the capacity of
    the buffer it arrived in: the stream is followed by whatever the buffer held before, and every
    block is active.  The integer deltas come from quant_predict, as in that schedule
    (HomComp/src/cuda_awareallreduce.cu:212-235)."""
    x, y, eb, _ = operands(gen, orc, name, n)
    ca, cb = orc.compress(x, eb), orc.compress(y, eb)
    cap = orc.max_stream_bytes(n)
    rng = np.random.default_rng(3)
    buf_a = rng.integers(0, 256, cap, dtype=np.uint8)
    buf_a[:ca.size] = ca
    buf_b = rng.integers(0, 256, cap, dtype=np.uint8)
    buf_b[:cb.size] = cb
    same_f32(emu.run("decompress", n, eb, buf_a, dtype=np.float32), orc.decompress(buf_a, n, eb, cmp_size=cap), "decompress")
    deltas = emu.run("quant_predict", n, eb, y, dtype=np.int32)
    assert np.array_equal(deltas, orc.quant_predict(y, eb)), "quant_predict"
    # (the two sums differ in the block that holds the end of a ragged operand: the float path's first
    # padded element has the delta 0 - q[n-1], the precomputed deltas end with zeros)
    want = orc.hom_sum_i32(buf_a, deltas, cmp_in_size=cap)
    want_f32 = orc.hom_sum_f32(buf_a, y, eb, cmp_in_size=cap)
    for kind in (0, 1):
        for groups, budget, slots in ((1, Emu.BUDGETS[1], 2), (3, Emu.BUDGETS[3], 3)):
            cfg = dict(kind=kind, groups=groups, budget=budget, slots=slots)
            same(emu.run("hom_sum_i32", n, eb, buf_a, deltas, **cfg), want, f"hom_sum_i32 kind {kind} {groups}/{budget}/{slots}")
            same(emu.run("hom_sum_f32", n, eb, buf_a, y, **cfg), want_f32, f"hom_sum_f32 kind {kind} {groups}/{budget}/{slots}")
    for kind in (1, 2):
        same(emu.run("hom_add", n, eb, buf_a, buf_b, kind=kind), orc.hom_add(buf_a, buf_b, n, size_a=cap, size_b=cap), f"hom_add kind {kind}")


def test_partial_sums_of_a_ring(emu, orc, gen):
    """Eight operands summed one after the other, the way a ring's reduce-scatter does: the plane
    counts grow with every step, so the later steps leave the few-plane path tile by tile."""
    n = 32768 + 5000
    xs = [gen.smooth_np(n, seed=s) for s in range(1, 9)]
    eb = bound_of(orc, 2e-4, *xs)
    want = orc.compress(xs[0], eb)
    got = emu.run("compress", n, eb, xs[0])
    same(got, want, "compress")
    for step, x in enumerate(xs[1:], 1):
        want = orc.hom_sum_f32(want, x, eb)
        got = emu.run("hom_sum_f32", n, eb, got, x, kind=1, groups=2)
        same(got, want, f"step {step}")
    other = orc.compress(xs[1], eb)
    for kind in (1, 2):
        same(emu.run("hom_add", n, eb, got, other, kind=kind), orc.hom_add(want, other, n), f"hom_add kind {kind} on the ring's sum")


def test_quant_predict_and_value_range(emu, orc, gen):
    for n in (1, 5, 4099, 70001):
        x, _, eb, _ = operands(gen, orc, "smooth_fine", 70001)
        x = x[:n].copy()
        got = emu.run("quant_predict", n, eb, x, dtype=np.int32)
        assert np.array_equal(got, orc.quant_predict(x, eb)), f"quant_predict n={n}"
        lo, hi = orc.value_range(x)
        got = emu.run("value_range", n, eb, x, groups=3, dtype=np.float32)
        assert got[0] == lo and got[1] == hi, f"value_range n={n}"


@pytest.mark.parametrize("op", ["compress", "hom_sum_f32"])
def test_a_grid_larger_than_the_device_holds(emu, orc, gen, op):
    """Six data workgroups and the scan server behind them on a device that holds three workgroups
    at a time: the first three wait for a server that cannot start before two of them have ended.
    Every wait ends at its bound, every workgroup runs to its end without touching memory that is
    not its own (any such access ends the run with another status), and the error word is raised;
    the same launch on a device that holds it gives the oracle's bytes."""
    n = 48 * 4096 + 77
    x, y = gen.smooth_np(n, 7), gen.smooth_np(n, 8)
    eb = bound_of(orc, 1e-5, x, y)
    sa = orc.compress(x, eb)
    a, b, want = (x, None, sa) if op == "compress" else (sa, y, orc.hom_sum_f32(sa, y, eb))
    report = emu.run(op, n, eb, a, b, groups=6, env={"EMU_RESIDENT": "3", "EMU_SPIN_LIMIT": "20"}, expect=5)
    assert "the kernels raised the error word" in report and "abnormally" not in report, report
    same(emu.run(op, n, eb, a, b, groups=6, env={"EMU_SPIN_LIMIT": "20000"}), want, "with the whole grid on the device")
