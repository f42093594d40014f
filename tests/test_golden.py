"""Golden fixture of the 1M-element smooth workload (tests/golden/config1.json): the CPU suite
checks that generator and oracle still reproduce it; the GPU suite checks the HIP kernels
against the same hashes."""
import hashlib
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.fixture(scope="module")
def fx():
    with open(os.path.join(HERE, "golden", "config1.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def inputs(fx, gen):
    x, y = gen.smooth_np(fx["n"], seed=1), gen.smooth_np(fx["n"], seed=2)
    eb = np.frombuffer(bytes.fromhex(fx["eb_abs_hex"]), np.float32)[0]
    return x, y, eb


def test_generator_is_reproducible(fx, inputs):
    x, y, _ = inputs
    assert sha(x) == fx["sha256_input"] and sha(y) == fx["sha256_input2"]


def test_oracle_reproduces_golden(fx, inputs, orc):
    x, y, eb = inputs
    mn, mx = orc.value_range(x)
    assert orc.rel_to_abs(1e-4, mn, mx) == eb
    s = orc.compress(x, eb)
    hb = fx["header_bytes"]
    assert s.size == fx["stream_len"] and orc.header_bytes(fx["n"]) == hb
    assert sha(s[:hb]) == fx["sha256_header"] and sha(s) == fx["sha256_stream"]
    assert s[hb:hb + 256].tolist() == fx["stream_head"] and s[-256:].tolist() == fx["stream_tail"]
    hist = np.bincount(s[:hb], minlength=256)
    assert {str(k): int(v) for k, v in enumerate(hist) if v} == fx["header_histogram"]
    dec = orc.decompress(s, fx["n"], eb)
    assert sha(dec) == fx["sha256_decompressed"]
    # round trip honours the bound (|err| <= eb up to float32 rounding)
    assert np.abs(dec.astype(np.float64) - x).max() <= float(eb) * 1.001
    h = orc.hom_sum_f32(s, y, eb)
    assert h.size == fx["hom_sum_len"] and sha(h) == fx["sha256_hom_sum"]


@pytest.mark.gpu
def test_gpu_reproduces_golden(fx, inputs, pkg, cuda):
    from gpu_util import Gpu
    x, y, eb = inputs
    g = Gpu(pkg, cuda, fx["n"])
    try:
        s = g.compress(x, eb)
        assert s.size == fx["stream_len"] and sha(s) == fx["sha256_stream"]
        assert sha(g.decompress(s, fx["n"], eb)) == fx["sha256_decompressed"]
        h = g.hom_sum_f32(s, y, eb)
        assert h.size == fx["hom_sum_len"] and sha(h) == fx["sha256_hom_sum"]
    finally:
        g.close()
