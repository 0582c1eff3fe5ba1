"""The reference's known-answer vectors through the C ABI on the GPU."""
import pytest

import kat_cases
from adam_amd import adamah as A
from gpu_util import note

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", kat_cases.ALL, ids=lambda f: f.__name__)
def test_hip_kat(hip, case):
    note(case.__name__)
    case(hip, A)
