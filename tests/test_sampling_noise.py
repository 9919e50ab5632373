"""The map from random bits to the Gumbel noise of temperature sampling, as the sampling kernel and its plain
statement (``emulated_kernels.gumbel_from_bits``) both compute it. The reference draws with ``categorical``
(/root/reference/src/levanter/layers/sampler.py:73), which cannot return an entry of probability zero: no entry's
noise may be infinite, whatever the bits are."""
import numpy as np

from emulated_kernels import gumbel_from_bits, gumbel_noise, philox4x32_10, uniform_from_bits


def test_uniform_is_strictly_inside_the_unit_interval_at_the_ends_of_the_range():
    bits = np.array([0xFFFFFFFF, 0, 0xFFFFFEFF, 0xFFFFFE00, 0x1FF, 0x200], dtype=np.uint32)
    u = uniform_from_bits(bits)
    assert u.dtype == np.float32
    assert (u > 0).all() and (u < 1).all(), u
    # exact values: the sums are float32 numbers, nothing rounds
    assert float(u[0]) == 1.0 - 2.0 ** -24 and float(u[1]) == 2.0 ** -24
    assert np.isfinite(gumbel_from_bits(bits)).all()


def test_every_possible_value_gives_finite_noise():
    """All 2^23 values that the map can see (it uses the top 23 bits)."""
    worst_low, worst_high = np.inf, -np.inf
    for start in range(0, 1 << 23, 1 << 21):
        top = np.arange(start, start + (1 << 21), dtype=np.uint32)
        u = uniform_from_bits(top << np.uint32(9))
        assert (u > 0).all() and (u < 1).all()
        g = gumbel_from_bits(top << np.uint32(9))
        assert np.isfinite(g).all()
        worst_low, worst_high = min(worst_low, float(g.min())), max(worst_high, float(g.max()))
    # -log(-log(2^-24)) and -log(-log(1 - 2^-24))
    assert abs(worst_low - (-np.log(24 * np.log(2.0)))) < 1e-4
    assert abs(worst_high - 24 * np.log(2.0)) < 0.1


def test_the_draw_that_once_rounded_up_to_one():
    """Key (1, 5), position 522, vocabulary 50,257: entry 21194 draws the largest 24-bit value. With 24 bits plus one half
    the uniform rounded to 1.0 and the noise to +inf, so that entry was sampled whatever the logits were."""
    g = np.uint64(21194 // 4)
    outs = philox4x32_10(np.array([g]), np.array([522], dtype=np.uint64), np.array([0], dtype=np.uint64),
                         np.array([0], dtype=np.uint64), 1, 5)
    bits = np.uint32(outs[21194 % 4][0])
    assert bits >> np.uint32(8) == 0xFFFFFF
    noise = gumbel_noise(1, 5, 522, 50257).numpy()
    assert np.isfinite(noise).all()
    assert int(noise.argmax()) == 21194 and 16.0 < float(noise[21194]) < 17.0


def test_noise_over_many_counters_is_finite_and_has_the_gumbel_mean():
    """2^22 consecutive counters of one key (16.8 million draws): finite, mean = Euler's constant, variance = pi^2 / 6."""
    total, total_sq, n = 0.0, 0.0, 0
    for start in range(0, 1 << 22, 1 << 19):
        c = np.arange(start, start + (1 << 19), dtype=np.uint64)
        z = np.zeros_like(c)
        outs = philox4x32_10(c, z + np.uint64(3), z, z, 77, 99)
        g = gumbel_from_bits(np.stack(outs, 1).reshape(-1).astype(np.uint32)).astype(np.float64)
        assert np.isfinite(g).all()
        total, total_sq, n = total + g.sum(), total_sq + (g * g).sum(), n + g.size
    mean = total / n
    var = total_sq / n - mean * mean
    assert abs(mean - 0.5772156649) < 2e-3
    assert abs(var - np.pi ** 2 / 6) < 5e-3
