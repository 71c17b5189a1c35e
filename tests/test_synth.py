"""The benchmark's counter-based generator (raft_amd/bench/synth.py): the tensor form and the
numpy form of every stream agree, so any element of a benchmark input can be recomputed on the
host from (seed, index)."""
import numpy as np
import pytest

from raft_amd.bench import synth


def _check(device):
    n = 70001
    idx = np.arange(n)
    for seed in (0, 2, 3, 7, 7921):
        assert np.array_equal(synth.uniform_device(seed, n, device).cpu().numpy(),
                              synth.uniform_host(seed, idx))
        assert np.array_equal(synth.int8_device(seed, n, device).cpu().numpy(),
                              synth.int8_host(seed, idx))
        got = synth.normal_device(seed, n, 3.0, 2.0, device).cpu().numpy()
        exp = synth.normal_host(seed, idx, 3.0, 2.0)
        assert np.abs(got - exp).max() <= 1e-5  # log / cos of two libraries
    # any slice of a long stream from its indices alone
    far = np.arange(1 << 33, (1 << 33) + 1000, dtype=np.uint64)
    u = synth.uniform_host(5, far)
    assert u.min() >= -1.0 and u.max() < 1.0 and len(np.unique(u)) > 990


def test_streams_agree_on_cpu():
    _check("cpu")
    # distribution sanity: a stream that ignored its counter or its seed would fail these
    u = synth.uniform_host(0, np.arange(200000))
    assert abs(u.mean()) < 0.01 and abs(u.std() - 1 / np.sqrt(3)) < 0.01
    g = synth.normal_host(3, np.arange(200000), 3.0, 2.0)
    assert abs(g.mean() - 3.0) < 0.02 and abs(g.std() - 2.0) < 0.02
    b = synth.int8_host(5, np.arange(200000))
    assert b.min() == -128 and b.max() == 127 and abs(b.astype(np.float64).mean()) < 1.0
    assert not np.array_equal(synth.uniform_host(1, np.arange(100)), synth.uniform_host(2, np.arange(100)))


def test_chunked_generation_is_seamless(monkeypatch):
    monkeypatch.setattr(synth, "_CHUNK", 1000)
    assert np.array_equal(synth.uniform_device(2, 5500, "cpu").numpy(),
                          synth.uniform_host(2, np.arange(5500)))


@pytest.mark.gpu
def test_streams_agree_on_gpu():
    _check("cuda")
