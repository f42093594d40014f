"""The gpu-marked parity tests run as they are (tests/test_gpu_parity.py, the same functions) with the library built for the host
(libhomcomp_emu.so, tests/emu) behind the same binding and helper: crafted streams of every plane
count, mode and outlier width, the bit-plane paths, payloads of random bytes under valid headers,
zero blocks, special values, empty input, truncated sizes, unaligned stream pointers, ragged
lengths, random mixtures, a graph replayed with eager calls between the replays; the plain
codec's tests, the tile offsets' (a recorded chain of ring steps among them) and the
allocation-free entry's (arguments, nothing allocated, recorded into a graph) likewise
(tests/test_gpu_plain.py, test_gpu_tile_offsets.py, test_zz_no_alloc.py)."""
import os
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import test_gpu_parity as parity  # noqa: E402
import test_gpu_plain as plain  # noqa: E402
import test_gpu_tile_offsets as tile_offsets  # noqa: E402
import test_zz_no_alloc as no_alloc  # noqa: E402
from gpu_util import Gpu  # noqa: E402


@pytest.fixture()
def world(emulated):
    """(the helper on a workspace of the emulated library, the binding, the torch stand-in)"""
    binding, harness = emulated
    t = harness.EmuTorch(binding.lib())
    g = Gpu(binding, t, parity.MAX_N)
    yield g, binding, t
    g.close()
    t.release()


@pytest.mark.parametrize("kind,n,mode,val", parity.CASES)
def test_compress_decompress(world, orc, gen, kind, n, mode, val):
    parity.test_compress_decompress(world[0], orc, gen, kind, n, mode, val)


@pytest.mark.parametrize("kind,n,mode,val", parity.CASES[:13])
def test_hom_sums(world, orc, gen, kind, n, mode, val):
    parity.test_hom_sums(world[0], orc, gen, kind, n, mode, val)


def test_every_rate_and_mode(world, orc):
    parity.test_every_rate_and_mode(world[0], orc)


def test_few_planes_per_step(world, orc):
    parity.test_few_planes_per_step(world[0], orc)


def test_sums_in_the_bit_plane_domain(world, orc):
    parity.test_sums_in_the_bit_plane_domain(world[0], orc)


@pytest.mark.parametrize("max_planes", [6, 31])
def test_arbitrary_payload_bytes(world, orc, max_planes):
    parity.test_arbitrary_payload_bytes(world[0], orc, max_planes)


def test_zero_incoming_blocks(world, orc, gen):
    parity.test_zero_incoming_blocks(world[0], orc, gen)


@pytest.mark.parametrize("special", ["zeros", "constant", "nan_inf", "huge", "alternating"])
def test_special_values(world, orc, special):
    parity.test_special_values(world[0], orc, special)


def test_empty(world):
    parity.test_empty(world[0], world[1], world[2])


def test_truncated_stream_size(world, orc, gen):
    parity.test_truncated_stream_size(world[0], orc, gen)


@pytest.mark.parametrize("offset", [1, 2, 3, 5, 8, 15])
def test_unaligned_stream_pointers(world, orc, gen, offset):
    parity.test_unaligned_stream_pointers(world[0], orc, gen, offset)


@pytest.mark.parametrize("seed", range(12))
def test_random_mixtures(world, orc, gen, seed):
    parity.test_random_mixtures(world[0], orc, gen, seed)


def test_argument_errors(world):
    parity.test_argument_errors(world[0], world[1], world[2])


def test_value_range(world, orc, gen):
    parity.test_value_range(world[0], orc, gen, world[1])


def test_workspace_reuse_many_calls(world, orc, gen):
    parity.test_workspace_reuse_many_calls(world[0], orc, gen)


@pytest.mark.parametrize("grid_percent", [1])
def test_many_rounds_and_small_grids(world, orc, gen, monkeypatch, grid_percent):
    parity.test_many_rounds_and_small_grids(world[1], world[2], orc, gen, monkeypatch, grid_percent)


@pytest.mark.parametrize("stage,slots", [("small", 4)])
def test_lds_budgets_and_deferral_depths(world, orc, gen, monkeypatch, stage, slots):
    parity.test_lds_budgets_and_deferral_depths(world[1], world[2], orc, gen, monkeypatch, stage, slots)


def test_lds_budget_follows_the_data(world, orc, gen):
    parity.test_lds_budget_follows_the_data(world[1], world[2], orc, gen)


@pytest.mark.parametrize("forced", [None, "2"])
def test_sum_kernel_follows_the_incoming_tiles(world, orc, gen, monkeypatch, forced):
    parity.test_sum_kernel_follows_the_incoming_tiles(world[1], world[2], orc, gen, monkeypatch, forced)


@pytest.mark.parametrize("forced", [None, "2", "3"])
def test_stream_plus_stream_wide_blocks(world, orc, monkeypatch, forced):
    parity.test_stream_plus_stream_wide_blocks(world[1], world[2], orc, monkeypatch, forced)


@pytest.mark.parametrize("tiles,offset", [(2049, 5)])
def test_offsets_prepass_sizes(world, orc, gen, tiles, offset):
    parity.test_offsets_prepass_sizes(world[1], world[2], orc, gen, tiles, offset)


# ---- tests/test_gpu_plain.py
@pytest.mark.parametrize("kind,n,rel", [c for c in plain.CASES if c[1] <= 1 << 18])
def test_plain_codec(world, orc, gen, kind, n, rel):
    plain.test_plain_codec(world[0], orc, gen, kind, n, rel)


def test_plain_equals_outlier_codec_without_outlier_blocks(world, orc, gen):
    plain.test_plain_equals_outlier_codec_without_outlier_blocks(world[0], orc, gen)


def test_plain_unaligned_and_saturated(world, orc):
    plain.test_plain_unaligned_and_saturated(world[0], orc)


def test_plain_decoder_reads_no_further_than_the_stream(world, orc, gen):
    plain.test_plain_decoder_reads_no_further_than_the_stream(world[0], orc, gen)


# ---- tests/test_gpu_tile_offsets.py
@pytest.mark.parametrize("kind,n,rel", [c for c in tile_offsets.CASES if c[1] <= 1 << 18])
def test_offsets_written_and_taken(world, orc, gen, kind, n, rel):
    tile_offsets.test_offsets_written_and_taken(world[1], world[2], orc, gen, kind, n, rel)


# ---- tests/test_zz_no_alloc.py
def test_static_entry_limits_and_arguments(world):
    no_alloc.test_static_entry_limits_and_arguments(world[1], world[2])


# ---- graphs: the model records the launches a capture makes and runs them again at every replay; an
#      allocation, a copy or a memset while a capture is under way would end the run with a report
def test_graph_replay(world, orc, gen):
    parity.test_graph_replay(world[1], world[2], orc, gen)


def test_ring_steps_recorded_with_offsets(world, orc, gen):
    tile_offsets.test_ring_steps_recorded_with_offsets(world[1], world[2], orc, gen)


def test_static_entry_in_a_graph(world, orc, gen):
    no_alloc.test_static_entry_in_a_graph(world[1], world[2], orc, gen)


def test_static_entry_allocates_nothing(world, orc, gen):
    no_alloc.test_static_entry_allocates_nothing(world[1], world[2], orc, gen)


# ---- several callers at once: on the model every launch runs alone, whichever host thread makes it, so
#      what this exercises here is the library's host side (its locks, the per-device state, the
#      workspaces created while other threads launch), not the overlap of kernels.  (The test with two
#      streams passes on the model too, HOMCOMP_CPU_MODEL=1, but is a minute of sequential calls there.)
def test_workspaces_created_while_other_threads_launch(world, orc, gen):
    parity.test_workspaces_created_while_other_threads_launch(world[1], world[2], orc, gen)
