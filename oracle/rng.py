"""Integer-exact restatement of the reference device RNG.  TEST INFRASTRUCTURE ONLY.

Follows sklearn_numba_dpex/common/random.py:
  * SplitMix64 seeding of state 0                      random.py:196-204, 245-250
  * xoroshiro128++ next (rotl 17 / 49 / 28, shift 21)  random.py:269-292
  * 2**64 jump polynomial                               random.py:206-230
  * state i = state i-1 jumped once                     random.py:256-261
  * uint64 -> [0, 1) float32 (>>40, * 2**-24) and float64 (>>11, * 2**-53)
                                                        random.py:78-104
  * seed drawn from a numpy RandomState                 random.py:156-157

Pinned by: the raw uint64 golden vectors for seed 42 and for seed 42 after one jump,
and the ten float32 uniforms, held in the reference's
common/tests/test_random.py:35-46, 54-65, 82-96 (tests/test_oracle_rng.py).
"""

import numpy as np

_M64 = (1 << 64) - 1


def _rotl(x, k):
    return ((x << k) | (x >> (64 - k))) & _M64


def splitmix64_next(state):
    state = (state + 0x9E3779B97F4A7C15) & _M64
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return state, z ^ (z >> 31)


class Xoroshiro128pp:
    """A bank of xoroshiro128++ generators, `states[i]` = [s0, s1] as Python ints."""

    JUMP = (0x2BD7A6A6E99C2DDC, 0x0992CCAF6A6FCA05)

    def __init__(self, n_states, seed, subsequence_start=0):
        seed = int(seed) & _M64
        sm, s0 = splitmix64_next(seed)
        _, s1 = splitmix64_next(sm)
        self.states = [[s0, s1]]
        for _ in range(subsequence_start):
            self._jump(0)
        for idx in range(1, n_states):
            self.states.append(list(self.states[idx - 1]))
            self._jump(idx)

    def next_raw(self, idx=0):
        s0, s1 = self.states[idx]
        result = (_rotl((s0 + s1) & _M64, 17) + s0) & _M64
        s1 ^= s0
        self.states[idx][0] = _rotl(s0, 49) ^ s1 ^ ((s1 << 21) & _M64)
        self.states[idx][1] = _rotl(s1, 28)
        return result

    def _jump(self, idx):
        s0 = s1 = 0
        for const in self.JUMP:
            for b in range(64):
                if const & (1 << b):
                    s0 ^= self.states[idx][0]
                    s1 ^= self.states[idx][1]
                self.next_raw(idx)
        self.states[idx][0] = s0
        self.states[idx][1] = s1

    def uniform(self, idx, dtype):
        return raw_to_uniform(self.next_raw(idx), dtype)


def raw_to_uniform(raw, dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return np.float32(raw >> 40) * (np.float32(1) / np.float32(1 << 24))
    if dtype == np.float64:
        return np.float64(raw >> 11) * (np.float64(1) / np.float64(1 << 53))
    raise ValueError(f"unsupported dtype {dtype}")


def seed_from_random_state(random_state):
    """The uint64 seed the reference draws from a numpy RandomState."""
    return int(random_state.randint(0, np.iinfo(np.int64).max - 1))
