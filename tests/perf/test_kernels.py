"""One timed comparison per case of the reference's kernel-level perf suite (tests/perf/test_primitives.py,
test_fused.py).  Nothing is asserted about the ratio — the suite tracks performance; a failure means the compile,
the run or the accuracy check against eager failed."""

import pytest

from tests.perf.cases import CASES

pytestmark = pytest.mark.perf


@pytest.mark.parametrize("case", CASES, ids=lambda c: c.name)
def test_kernel_perf(case, bench_pair):
    bench_pair(case)
