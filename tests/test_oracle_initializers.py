"""CPU checks of the row initializers.

The oracle restates libstdc++'s minstd_rand0 / generate_canonical / normal_distribution<float> by hand; pins:
  * the C++ standard's known answer for minstd_rand0 (10000th value from seed 1 is 1043618065),
  * what the reference's own test asserts on initialised rows (emb_cache_test.cpp:433-455: constant columns equal the
    constant, truncated columns lie within two standard deviations, normal columns have the configured mean/stddev),
  * a Kolmogorov-Smirnov test of the normal stream against the normal CDF,
  * the std classes themselves (std::default_random_engine + std::normal_distribution<float>, what the reference's
    initializers call) give the oracle's stream bit for bit,
  * the host library's initializers, which produce the same stream in pieces on several threads (the engine jumps
    ahead by modular exponentiation), give the same bits, across piece and refill boundaries.
"""
import numpy as np
from scipy import stats

import oracle
from recsdk_amd import host

C, N, TN = oracle.INIT_CONSTANT, oracle.INIT_RANDOM_NORMAL, oracle.INIT_TRUNCATED_NORMAL


def test_minstd_rand0_standard_known_answer():
    assert int(oracle.minstd_rand0(1, 10000)[-1]) == 1043618065
    assert int(oracle.minstd_rand0(0, 1)[0]) == 16807          # seed 0 is replaced by 1


def test_reference_test_assertions():
    # SimpleCreateTable (emb_cache_test.cpp:51-90): normal(0, 0.05) | constant 0.233 | truncated normal(0, 0.05)
    emb = 13
    descs = [(N, 0, emb, 0.0, 0.05, 0, 1.0), (C, emb, emb, 0.233, 0.0, 0, 1.0), (TN, 2 * emb, emb, 0.0, 0.05, 0, 1.0)]
    rows = oracle.Initializer(descs).generate(4000, 3 * emb)
    assert abs(rows[:, :emb].mean()) < 0.05 * 4 / np.sqrt(4000 * emb)
    assert abs(rows[:, :emb].std() - 0.05) < 0.05 * 0.02
    assert np.all(np.abs(rows[:, emb:2 * emb] - 0.233) <= 1e-6)
    assert np.all(np.abs(rows[:, 2 * emb:]) <= 0.1 + 1e-6)
    assert rows[:, 2 * emb:].std() < 0.05                         # truncation narrows the distribution


def test_normal_stream_is_normal():
    x = oracle.Initializer([(N, 0, 1, 1.5, 2.0, 7, 1.0)]).generate(20000, 1)[:, 0]
    assert stats.kstest((x - 1.5) / 2.0, "norm").pvalue > 1e-3
    y = oracle.Initializer([(N, 0, 1, 1.5, 2.0, 7, 3.0)]).generate(20000, 1)[:, 0]
    np.testing.assert_array_equal(y, np.float32(3.0) * x)          # init_k multiplies the drawn value


def test_limits_are_clamped():
    r = oracle.Initializer([(C, 0, 2, 5e9, 0.0, 0, 20000.0)]).generate(1, 2)
    np.testing.assert_array_equal(r, np.full((1, 2), np.float32(1e9) * np.float32(10000.0)))


def test_library_initializers_match_oracle_bits():
    descs = [(N, 0, 8, 0.1, 0.7, 11, 1.0), (C, 8, 4, -2.5, 0.0, 0, 2.0), (TN, 12, 8, 0.0, 0.05, 3, 1.0),
             (N, 20, 4, 0.0, 1.0, 11, 0.5)]
    want = oracle.Initializer(descs)
    got = host.Initializer(descs)
    for rows in (1, 3, 500):   # the generators keep their state from call to call
        np.testing.assert_array_equal(got.generate(rows, 24), want.generate(rows, 24))
    np.testing.assert_array_equal(got.generate(2, 32, fill=9.0)[:, 24:], np.full((2, 8), 9.0, np.float32))


def test_oracle_stream_is_the_std_classes_stream():
    for seed, mean, std in [(0, 0.0, 1.0), (7, 1.5, 2.0), (123456789, -0.25, 0.01), (2147483647, 0.0, 0.05)]:
        want = oracle.std_normal(seed, mean, std, 200001)
        got = oracle.Initializer([(N, 0, 1, mean, std, seed, 1.0)]).generate(200001, 1)[:, 0]
        np.testing.assert_array_equal(got, want)


def test_library_stream_matches_across_piece_and_refill_boundaries():
    """1.3 M values per call and several calls: the library cuts the attempts into pieces of 65536 for its threads and
    refills its buffer between calls; odd row widths leave a saved value of the polar method pending at every boundary"""
    descs = [(N, 0, 13, 0.0, 0.01, 5, 1.0), (TN, 13, 7, 0.0, 0.05, 9, 1.0), (C, 20, 1, 0.1, 0.0, 0, 1.0)]
    want = oracle.Initializer(descs)
    got = host.Initializer(descs)
    for rows in (100000, 1, 37, 250000, 3):
        np.testing.assert_array_equal(got.generate(rows, 21), want.generate(rows, 21))
    # and the stream itself against the std classes
    one = host.Initializer([(N, 0, 1, 0.0, 0.01, 5, 1.0)]).generate(1_000_003, 1)[:, 0]
    np.testing.assert_array_equal(one, oracle.std_normal(5, 0.0, 0.01, 1_000_003))
