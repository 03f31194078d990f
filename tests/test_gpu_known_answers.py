"""The reference's known-answer tests for the hot path, run through the C ABI on the GPU."""
import pytest

import known_answer_cases as kac

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", kac.CASES, ids=lambda f: f.__name__[5:])
def test_known_answer(case, gc):
    case(gc)


@pytest.mark.parametrize("name", kac.ELEMENTWISE_NAMES)
def test_elementwise_known_answer(name, gc):
    kac._elementwise(gc, name)
