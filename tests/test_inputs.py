"""The deterministic workload generator (kernelcodegen_amd/inputs.py)."""
import numpy as np

from kernelcodegen_amd import inputs


def _splitmix_scalar(x):
    mask = (1 << 64) - 1
    x = (x + 0x9E3779B97F4A7C15) & mask
    z = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    return z ^ (z >> 31)


def test_uniform_matches_scalar_definition():
    seed, tid = 0xC0DE0001, 1
    u = inputs.uniform((5, 7), seed, tid).ravel()
    for i in (0, 1, 17, 34):
        z = _splitmix_scalar(seed ^ (tid << 56) ^ i)
        assert u[i] == np.float32((z >> 40) / 8388608.0 - 1.0)
    assert u.min() >= -1.0 and u.max() < 1.0


def test_splitmix_known_answer():
    # First output of the reference SplitMix64 stream seeded with 0
    # (state 0 + golden gamma, then the finaliser): 0xE220A8397B1DCDAF.
    assert _splitmix_scalar(0) == 0xE220A8397B1DCDAF
    assert int(inputs._mix(np.array([0], dtype=np.uint64))[0]) == 0xE220A8397B1DCDAF


def test_counter_based_slices_agree():
    a = inputs.normal((1000,), 5, 2)
    b = inputs.normal((4, 250), 5, 2).ravel()
    assert np.array_equal(a, b)
    big = inputs.normal((inputs._CHUNK + 100,), 5, 2)      # crosses a chunk boundary
    assert np.array_equal(big[:1000], a)
    assert not np.array_equal(inputs.normal((1000,), 5, 1), a)
    assert not np.array_equal(inputs.normal((1000,), 6, 2), a)


def test_moments():
    n = inputs.normal((400000,), 9, 0)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1) < 0.01
    w = inputs.normal((400000,), 9, 1, std=0.02)
    assert abs(w.std() - 0.02) < 2e-4
    u = inputs.uniform((400000,), 9, 0)
    assert abs(u.mean()) < 0.01 and abs(u.var() - 1 / 3) < 0.01


def test_bf16_round_trip():
    x = inputs.normal((4096,), 3, 0)
    b = inputs.to_bf16_bits(x)
    back = inputs.bf16_bits_to_f32(b)
    assert np.all(np.abs(back - x) <= np.abs(x) * 2.0 ** -8)
    assert np.array_equal(inputs.to_bf16_bits(back), b)


def test_config_shapes():
    c0 = inputs.config_inputs(0)
    assert c0["A"].shape == (4096, 1024) and c0["B"].shape == (1024, 2048)
    c2 = inputs.config_inputs(2)
    assert c2["A"].shape == (32768, 768) and abs(c2["B"].std() - 0.02) < 1e-3
