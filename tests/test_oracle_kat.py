"""The oracle against the reference's own known-answer vectors (CPU only)."""
import pytest

import kat_cases
import oracle.adamah_np as onp
from adam_amd import adamah as A


@pytest.mark.parametrize("case", kat_cases.ALL, ids=lambda f: f.__name__)
def test_oracle_kat(case):
    case(onp.NumpyAdamah(), A)
