"""The counter-based input generator (ark_amd/prng.py): known answers of splitmix64's mixing
function, agreement of the numpy and torch paths word for word, and the moments of what it draws."""
import numpy as np
import torch

from ark_amd import prng


def test_words_known_answers_and_backends_agree():
    # seed 0, element 0 mixes the golden-ratio constant alone: splitmix64's first output for state 0
    w = prng._words_numpy(0, 0, 4)
    assert int(w[0]) == 0xE220A8397B1DCDAF
    # element i of a stream does not depend on how many elements are drawn or where the draw starts
    assert int(prng._words_numpy(0, 3, 1)[0]) == int(w[3])
    for seed in (0, 1, 12345, 0x7FFFFFFF):
        a = prng._words_numpy(seed, 0, 1000)
        b = prng._words_torch(seed, 0, 1000, "cpu").numpy().view(np.uint64)
        assert np.array_equal(a, b)
        assert len(np.unique(a)) == 1000


def test_uniform_and_normal():
    u = prng.uniform(3, (1 << 16,), -1.0, 1.0)
    assert u.dtype == np.float32 and u.min() >= -1.0 and u.max() < 1.0
    assert abs(float(u.mean())) < 0.01 and abs(float(u.var()) - 1.0 / 3.0) < 0.01
    assert np.array_equal(u, prng.uniform(3, (1 << 16,), -1.0, 1.0, device="cpu").numpy())
    assert np.array_equal(u[:100], prng.uniform(3, (256, 256), -1.0, 1.0).reshape(-1)[:100])
    n = prng.normal(4, (1 << 16,), 0.0, 0.02)
    assert abs(float(n.mean())) < 5e-4 and abs(float(n.std()) - 0.02) < 5e-4
    assert np.all(np.isfinite(n))
    nt = prng.normal(4, (1 << 16,), 0.0, 0.02, device="cpu").numpy()
    assert np.abs(n - nt).max() <= 1e-7  # the same values up to the platform's log / cos
    assert prng.seed_of("C1", "A") != prng.seed_of("C1", "B") and prng.seed_of("C1", "A") == prng.seed_of("C1", "A")
