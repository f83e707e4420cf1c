"""The float32 path against its frozen vectors (tests/golden/*.json, written by tests/golden.py --update): every way
of running the fixed requests reproduces the recorded sha256 of every logit row.  What this notices and the tests
within one run cannot: a change of the float32 arithmetic from one version of the code to the next."""
import json

import pytest

import golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=golden.NAMES)
def frozen(request, gpu):
    name = request.param
    with open(golden.path_of(name)) as f:
        g = json.load(f)
    why_not = golden.check_environment(name, g)
    if why_not:
        pytest.skip("the frozen vectors were made by another compiler or for another GPU and say nothing here "
                    "(tests/golden.py --update --reason ... after the other tests pass): " + "; ".join(why_not))
    return name, g


def test_the_model_is_the_frozen_one(frozen):
    name, g = frozen
    assert not golden.check_model(name, g)


@pytest.mark.parametrize("use_graphs", [True, False], ids=["graphs", "eager"])
@pytest.mark.parametrize("plan", golden.PLANS)
def test_float32_logits_are_the_frozen_ones(frozen, plan, use_graphs):
    name, g = frozen
    msgs = golden.compare(name, g, plan, use_graphs)
    assert not msgs, (f"configuration {name}, {plan}, {'graphs' if use_graphs else 'eager'}: the float32 logits are not the "
                      f"frozen ones (a deliberate change of the arithmetic: tests/golden.py --update --reason ...):\n  "
                      + "\n  ".join(msgs))
