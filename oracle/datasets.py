"""The frozen data generators live with the package (they are inputs, not part of the oracle);
re-exported here for the tests that import them next to the oracle.
TEST INFRASTRUCTURE ONLY."""

from sklearn_numba_dpex_amd.datasets import config1, config2, config3, config4, config5  # noqa: F401
