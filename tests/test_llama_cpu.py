"""CPU checks of the host-side Llama helpers that feed both sides of every layer test."""
import math

import numpy as np

from ark_amd import llama


def test_precompute_freqs_cis_closed_form():
    """The rotary table is exp(i * t * theta^(-2j/d)) stored as interleaved (re, im) in
    [1, seq, 1, head_dim] (examples/llama/generator.py:20-27, layout model_test.py:379-384):
    hand-picked (t, j) against cos/sin evaluated independently, unit modulus everywhere, and the
    rotation property table[t] = table[1]^t."""
    d, seq, theta = 128, 2048, 10000.0
    tab = llama.precompute_freqs_cis(d, seq, theta)
    assert tab.shape == (1, seq, 1, d) and tab.dtype == np.float32
    tab = tab.reshape(seq, d)
    for t, j in [(0, 0), (0, 63), (1, 0), (1, 1), (1, 63), (7, 5), (100, 32), (2047, 0), (2047, 63), (1234, 17)]:
        ang = t * math.pow(theta, -2.0 * j / d)
        assert abs(tab[t, 2 * j] - math.cos(ang)) <= 1e-6, (t, j)
        assert abs(tab[t, 2 * j + 1] - math.sin(ang)) <= 1e-6, (t, j)
    re, im = tab[:, 0::2].astype(np.float64), tab[:, 1::2].astype(np.float64)
    assert np.abs(re * re + im * im - 1.0).max() <= 1e-6
    # position 0 is the identity rotation; frequency 0 turns by one radian per position
    assert np.all(re[0] == 1.0) and np.all(im[0] == 0.0)
    assert abs(math.atan2(im[3, 0], re[3, 0]) - 3.0) <= 1e-6
    # frequencies fall geometrically: the last pair turns theta^(-(d-2)/d) radians per position
    assert abs(math.atan2(im[1, 63], re[1, 63]) - theta ** (-(d - 2) / d)) <= 1e-7
    # t -> t + 1 is a multiplication by table[1]
    z = re + 1j * im
    assert np.abs(z[1:] - z[:-1] * z[1]).max() <= 1e-6


def test_causal_mask_layout():
    m = llama.causal_mask(5, -np.inf).reshape(5, 5)
    assert np.all(np.isneginf(m[np.triu_indices(5, k=1)]))
    assert np.all(m[np.tril_indices(5)] == 0)
