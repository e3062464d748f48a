"""The oracle's restatement of temperature sampling, pinned by what the mathematics fixes (CPU only)."""
import numpy as np


def test_splitmix64_known_answers(orc):
    """First three outputs of SplitMix64 seeded with 0 (the values every published implementation lists)."""
    g = 0x9E3779B97F4A7C15
    assert orc.splitmix64(0) == 0xE220A8397B1DCDAF
    assert orc.splitmix64(g) == 0x6E789E6AA1B965F4
    assert orc.splitmix64((2 * g) & ((1 << 64) - 1)) == 0x06C45D188009454F


def test_uniform_range_and_keys(orc):
    u = np.array([orc.sample_uniform(9, s, p) for s in range(4) for p in range(500)])
    assert u.min() >= 0.0 and u.max() < 1.0
    assert abs(u.mean() - 0.5) < 0.02 and abs(u.var() - 1 / 12) < 0.01
    assert len(set(u.tolist())) == u.size                       # (seed, sequence, position) keys do not collide here
    assert orc.sample_uniform(9, 1, 7) != orc.sample_uniform(10, 1, 7)
    assert orc.sample_uniform(9, 1, 7) == orc.sample_uniform(9, 1, 7)


def test_limits(orc):
    rng = np.random.default_rng(0)
    lg = rng.normal(size=257)
    best = int(np.argmax(lg))
    for u in (0.0, 0.3, 0.999999):
        assert orc.sample_token(lg, 1e-4, u) == best            # T -> 0: all the mass on the argmax
    assert orc.sample_token(lg, 1.0, 0.0) == 0                  # every probability is positive: u = 0 takes index 0
    assert orc.sample_token(lg, 1.0, 1.0 - 2.0 ** -53) == 256   # the largest u takes the last index
    picks = [orc.sample_token(lg, 0.7, u) for u in np.linspace(0, 1, 400, endpoint=False)]
    assert picks == sorted(picks)                               # inverse CDF: monotone in u
    flat = np.zeros(10)
    assert [orc.sample_token(flat, 1.0, (k + 0.5) / 10) for k in range(10)] == list(range(10))  # uniform: deciles


def test_frequencies_follow_the_softmax(orc):
    lg = np.array([0.2, -1.0, 1.5, 0.0, 0.7, -0.3, 2.0, -2.0])
    T, n = 0.8, 40000
    p = np.exp(lg / T) / np.exp(lg / T).sum()
    counts = np.bincount([orc.sample_token(lg, T, orc.sample_uniform(3, 0, i)) for i in range(n)], minlength=8)
    sigma = np.sqrt(n * p * (1 - p))
    assert np.all(np.abs(counts - n * p) < 5 * sigma), (counts, n * p)
