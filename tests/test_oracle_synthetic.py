"""The counter-based synthetic-data generator: the oracle's NumPy statement, its C twin and the
library's host-only key function agree; the distributions are what the benchmark configurations ask for."""
import ctypes as C
import os
import sys

import numpy as np

import mxopt_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "mlx-node_amd"))


def test_numpy_and_c_twin_agree(oracle_c):
    for dist, a, b in ((O.SYNTH_NORMAL, 1e-3, 0.0), (O.SYNTH_NORMAL_OUTLIERS, 1e-3, 100.0), (O.SYNTH_UNIFORM, 0.9, 1.1),
                       (O.SYNTH_GAUSSIAN, 1e-3, 0.0), (O.SYNTH_GAUSSIAN_OUTLIERS, 1e-3, 100.0)):
        for dt in ("f32", "bf16"):
            for first in (0, 7, 2 ** 40 + 3):
                x = O.synthetic(50021, dt, 0xDEADBEEF12345678, dist, a, b, first_index=first)
                y = oracle_c.fill_synthetic(50021, dt, 0xDEADBEEF12345678, dist, a, b, first_index=first)
                assert np.array_equal(x, y), (dist, dt, first)


def test_a_slice_is_the_same_as_the_middle_of_the_whole():
    whole = O.synthetic(10000, "bf16", 42, O.SYNTH_NORMAL, 0.02)
    assert np.array_equal(O.synthetic(100, "bf16", 42, O.SYNTH_NORMAL, 0.02, first_index=1234), whole[1234:1334])


def test_distributions():
    x = O.synthetic(4_000_000, "f32", 1, O.SYNTH_NORMAL, 1e-3).astype(np.float64)
    assert abs(x.mean()) < 3e-6 and abs(x.std() - 1e-3) < 2e-6 and np.abs(x).max() <= 3.47e-3
    assert abs(np.mean(np.abs(x) < 1e-3) - 0.669) < 0.005                    # bell shaped: 66.9 % within one sigma (a normal has 68.3 %)
    y = O.synthetic(4_000_000, "f32", 2, O.SYNTH_NORMAL_OUTLIERS, 1e-3, 100.0).astype(np.float64)
    assert abs(np.mean(np.abs(y) > 3.5e-3) - 0.0097) < 0.001                 # 1 % x100, a few of them still small
    assert abs(np.sqrt(np.mean(y * y)) - 1e-3 * np.sqrt(0.99 + 0.01 * 1e4)) < 2e-4
    u = O.synthetic(1_000_000, "f32", 3, O.SYNTH_UNIFORM, 0.9, 1.1)
    assert u.min() >= 0.9 and u.max() < 1.1 and abs(u.mean() - 1.0) < 2e-4
    assert len(np.unique(O.synthetic(100000, "f32", 4, O.SYNTH_UNIFORM, 0.0, 1.0))) > 99000
    # different streams are unrelated
    a, b = O.synthetic(100000, "f32", 10, 0, 1.0), O.synthetic(100000, "f32", 11, 0, 1.0)
    assert abs(np.corrcoef(a, b)[0, 1]) < 0.02


def test_gaussian_mode_is_a_normal_distribution_with_its_tails():
    """What the mathematics fixes: the committed quantile table against scipy's inverse normal CDF, the samples
    against the normal CDF (Kolmogorov-Smirnov), moments, and tail masses beyond 3.46 sigma -- where the
    four-uniform bell stops -- against erfc."""
    import math
    from scipy import stats
    from scipy.special import ndtri
    t = O.gauss_quantile_table()
    assert t.shape == (32, 33) and t.dtype == np.float32
    for k in (0, 1, 7, 20, 31):
        for j in (0, 5, 32):
            p = 2.0 ** -(k + 1) * (1 + j / 32)
            want = 0.0 if p == 1.0 else -ndtri(p / 2)
            assert abs(float(t[k, j]) - want) <= 1e-6 * max(want, 1.0), (k, j)
    assert (np.diff(t, axis=1) < 0).all() and np.array_equal(t[1:, 32], t[:-1, 0])      # decreasing, rows join up
    x = O.synthetic(8_000_000, "f32", 5, O.SYNTH_GAUSSIAN, 1.0).astype(np.float64)
    assert abs(x.mean()) < 1.5e-3 and abs(x.std() - 1.0) < 1.5e-3
    assert abs(stats.skew(x)) < 5e-3 and abs(stats.kurtosis(x)) < 1e-2
    assert stats.kstest(x[:2_000_000], "norm").pvalue > 1e-3
    for thr in (1.0, 2.0, 3.0, 3.46, 4.0):
        got, want = np.mean(np.abs(x) > thr), math.erfc(thr / math.sqrt(2))
        assert abs(got - want) < 4 * math.sqrt(want / x.size) + 1e-7, (thr, got, want)
    assert np.abs(x).max() > 4.8                                                        # far beyond the bell's 3.46
    assert O.synthetic(4, "f32", 5, O.SYNTH_GAUSSIAN, 2.5, first_index=10).tolist() == \
        (O.synthetic(4, "f32", 5, O.SYNTH_GAUSSIAN, 1.0, first_index=10) * np.float32(2.5)).tolist()
    y = O.synthetic(4_000_000, "f32", 6, O.SYNTH_GAUSSIAN_OUTLIERS, 1e-3, 100.0).astype(np.float64)
    assert abs(np.sqrt(np.mean(y * y)) - 1e-3 * np.sqrt(0.99 + 0.01 * 1e4)) < 3e-4
    # the extreme codes: u = 0 is taken as 1 (|x| = 6.3 sigma), u = 2^32 - 1 gives almost 0
    assert 6.2 < float(O._gauss_magnitude(np.array([0], np.uint64))[0]) < 6.4
    assert 0.0 <= float(O._gauss_magnitude(np.array([2 ** 32 - 1], np.uint64))[0]) < 1e-6


def test_key_function_matches_the_library():
    from mxopt import _lib
    lib = _lib.load()
    for args in ((0x5EED0001, 5, 0, 0, 0), (0x5EED0001, 5, 9, 3, 398), (2 ** 64 - 1, 0, 2 ** 31, 65535, 2 ** 32)):
        assert lib.mxopt_synthetic_key(*[C.c_uint64(v & (2 ** 64 - 1)) for v in args]) == O.synthetic_key(*args), args
    assert O.synthetic_key(1, 2, 3, 4, 5) != O.synthetic_key(1, 2, 3, 4, 6)


def test_known_answers_freeze_the_generator():
    """The definition must never drift: benchmark inputs of earlier runs stay reproducible.  Six elements of
    each distribution from one key, as bit patterns (the fifth element of the second row is a x100 outlier)."""
    key = O.synthetic_key(0x5EED0001, 5, 0, 3, 17)
    assert key == 0xF5409BCF2ED3FA2A
    normal = O.synthetic(6, "f32", key, O.SYNTH_NORMAL, 1e-3, 0.0, first_index=1000003)
    assert [int(v) for v in normal.view(np.uint32)] == [0xBA5FD61E, 0xB8FC2194, 0xB9FD7291, 0x3A934168, 0x39DCF0BE, 0x3A68FB4B]
    outliers = O.synthetic(6, "bf16", key, O.SYNTH_NORMAL_OUTLIERS, 1e-3, 100.0, first_index=1000003)
    assert [int(v) for v in outliers] == [0xBA60, 0xB8FC, 0xB9FD, 0x3A93, 0x3D2D, 0x3A69]
    gauss = O.synthetic(6, "f32", key, O.SYNTH_GAUSSIAN, 1e-3, 0.0, first_index=1000003)
    assert [int(v) for v in gauss.view(np.uint32)] == [0x3B1B608D, 0x39DE0DF6, 0x3A80B027, 0xBA724D5E, 0x39A76670, 0x3A9A274A]
    uniform = O.synthetic(6, "f32", key, O.SYNTH_UNIFORM, 0.9, 1.1, first_index=1000003)
    assert [int(v) for v in uniform.view(np.uint32)] == [0x3F66DAB6, 0x3F7799CB, 0x3F6EC035, 0x3F848C60, 0x3F799660, 0x3F6C8862]
