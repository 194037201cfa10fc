"""A fixed range of seeds of the random-case runner (tests/hostsim/fuzz.py): random shapes (half of
them at or next to a multiple of 32), masks, dtypes, batch sizes and call options of every operator
on the kernels' host build against the oracle.  The runner itself takes any range of seeds."""

import pytest

from tests.hostsim import fuzz


@pytest.mark.parametrize("seed", range(40))
def test_random_case(seed):
    what, e = fuzz.run_seed(seed)
    print(seed, what, e)


@pytest.mark.parametrize("family,seed", [("api", s) for s in range(8)] + [("wide_block", 3), ("template_block", 5)])
def test_random_case_of_family(family, seed):
    what, e = fuzz.run_seed(seed, family)
    print(seed, what, e)
