"""Pins the CPU checker (and the host-side autograd mirror) against the reference's own
known-answer tests for the hot path. No GPU involved."""
import pytest

import known_answer_cases as kac


@pytest.mark.parametrize("case", kac.CASES, ids=lambda f: f.__name__[5:])
def test_known_answer(case, oracle_ops):
    case(oracle_ops)


@pytest.mark.parametrize("name", kac.ELEMENTWISE_NAMES)
def test_elementwise_known_answer(name, oracle_ops):
    kac._elementwise(oracle_ops, name)
