"""CPU restatement of the reference KMeans path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this directory: it is the checker the
GPU results are compared with (tests, the smoke check, and the CPU-baseline leg
of the benchmark), never the thing that is measured or shipped.

Modules
-------
rng      xoroshiro128++ / SplitMix64 integer RNG      (reference common/random.py)
kmeans   Lloyd, labels, inertia, distances, kmeans++,
         relocation, centering, clustering helpers    (reference kmeans/drivers.py and
                                                        kmeans/kernels/*.py)
         (top-k, sums and argmin have no module here: the tests check them against
         numpy's sort / sum / argmin directly, as the reference's own tests do)
datasets frozen synthetic generators for the benchmark configurations

Pinning status (which independent evidence holds each function in place) is listed
at the top of each module.
"""
