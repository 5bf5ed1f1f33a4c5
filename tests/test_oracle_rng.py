"""The RNG restatements (oracle and the package's host RNG) against the golden vectors the
reference's tests hold (sklearn_numba_dpex/common/tests/test_random.py:35-46, 54-65, 82-96)."""

import numpy as np
import pytest

from oracle import rng as orng
from sklearn_numba_dpex_amd.common import random as prng

SEED42_RAW = [
    16756476715040848931, 6098722386207918385, 17541662578032534341, 3771828211556203317,
    6324094075403496319, 1696280121849217124, 9039151786603216578, 1834868434787995627,
    4294676528364711596, 5649342080498856832,
]
SEED42_JUMPED_RAW = [
    16052925335932940643, 13241858892588731496, 8234838429006980292, 1690280486132429899,
    6807031509475728656, 9789629428737685881, 8662181912786361632, 11992761958092131212,
    7748117140003924005, 5731413122647051604,
]
SEED42_F32 = np.array(
    [0.9083704, 0.33061236, 0.9509354, 0.20447117, 0.34282982, 0.09195548, 0.49001336, 0.09946841,
     0.23281485, 0.3062514], dtype=np.float32)


def test_oracle_raw_golden_vectors():
    g = orng.Xoroshiro128pp(1, 42)
    assert [g.next_raw() for _ in SEED42_RAW] == SEED42_RAW
    g = orng.Xoroshiro128pp(1, 42, subsequence_start=1)
    assert [g.next_raw() for _ in SEED42_JUMPED_RAW] == SEED42_JUMPED_RAW


def test_package_raw_golden_vectors():
    s = prng.create_xoroshiro128pp_states(1, seed=42)
    assert [prng.get_random_raw(s) for _ in SEED42_RAW] == SEED42_RAW
    s = prng.create_xoroshiro128pp_states(1, seed=42, subsequence_start=1)
    assert [prng.get_random_raw(s) for _ in SEED42_JUMPED_RAW] == SEED42_JUMPED_RAW


def test_state_i_is_state_0_jumped_i_times():
    # state 1 of a bank == state 0 of a generator started one subsequence later
    bank = prng.create_xoroshiro128pp_states(3, seed=42)
    assert [bank.next_raw(1) for _ in range(10)] == SEED42_JUMPED_RAW
    obank = orng.Xoroshiro128pp(3, 42)
    assert [obank.next_raw(1) for _ in range(10)] == SEED42_JUMPED_RAW
    # and the vectorised advance agrees with advancing each state alone
    a = prng.create_xoroshiro128pp_states(4, seed=7)
    b = prng.create_xoroshiro128pp_states(4, seed=7)
    for _ in range(5):
        all_at_once = a.next_raw_all()
        assert [int(v) for v in all_at_once] == [b.next_raw(i) for i in range(4)]


def test_uniform_float32_golden_and_float64_close():
    g = orng.Xoroshiro128pp(1, 42)
    got32 = np.array([g.uniform(0, np.float32) for _ in SEED42_F32], dtype=np.float32)
    np.testing.assert_allclose(got32, SEED42_F32, rtol=1e-7)
    g = orng.Xoroshiro128pp(1, 42)
    got64 = np.array([g.uniform(0, np.float64) for _ in SEED42_F32])
    np.testing.assert_allclose(got64, SEED42_F32, rtol=1e-6)
    s = prng.create_xoroshiro128pp_states(1, seed=42)
    pk = np.array([prng.raw_to_uniform(prng.get_random_raw(s), np.float32) for _ in SEED42_F32])
    np.testing.assert_array_equal(pk.astype(np.float32), got32)
    assert got32.min() >= 0 and got32.max() < 1


def test_uniform_histogram_is_flat():
    s = prng.create_xoroshiro128pp_states(64, seed=42)
    draws = np.concatenate([prng.raw_to_uniform(s.next_raw_all(), np.float64) for _ in range(4000)])
    hist, _ = np.histogram(draws, bins=np.linspace(0, 1, 6))
    assert np.all(np.abs(hist - draws.size / 5) < 0.02 * draws.size / 5)


def test_seed_from_random_state_matches_reference_recipe():
    rs = np.random.RandomState(3)
    expected = np.random.RandomState(3).randint(0, np.iinfo(np.int64).max - 1)
    assert orng.seed_from_random_state(rs) == expected
    a = prng.create_xoroshiro128pp_states(2, seed=np.random.RandomState(3))
    b = prng.create_xoroshiro128pp_states(2, seed=expected)
    np.testing.assert_array_equal(a.states, b.states)


def test_kpp_uniform_tables_agree():
    from oracle import kmeans as ok
    from sklearn_numba_dpex_amd.kmeans.drivers import kpp_uniforms

    for dtype in (np.float32, np.float64):
        seed = orng.seed_from_random_state(np.random.RandomState(5))
        start_o, table_o = ok.kpp_uniform_table(9, 4, seed, dtype)
        start_p, table_p = kpp_uniforms(9, 4, np.random.RandomState(5), dtype)
        assert start_o == start_p
        np.testing.assert_array_equal(table_o.astype(np.float64), table_p)
