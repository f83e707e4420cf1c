"""Every negative control of negative_controls.txt, on the GPU: the checks named for a control pass on
an unmutated scratch copy of the tree and fail on the copy that holds the control's bug."""
import os
import tempfile

import pytest

import negative_controls as nc

pytestmark = pytest.mark.gpu

CONTROLS = nc.read_table()


@pytest.fixture(scope="module")
def scratch(gpu):
    with tempfile.TemporaryDirectory(prefix="tuff_amd_negctl_") as tmp:
        tree = nc.make_scratch(os.path.join(tmp, "tree"))
        every = sorted({k for c in CONTROLS for k in c["checks"]})
        base = nc.run_checks(tree, every, None)
        broken = {k: base[k] for k in every if base[k] != "passed"}
        assert not broken, f"checks that do not pass on the unmutated tree: {broken}\n{base['_log']}"
        yield tree


@pytest.mark.parametrize("control", CONTROLS, ids=[c["id"] for c in CONTROLS])
def test_the_mutant_is_caught(scratch, control):
    nc.apply(control, scratch)
    try:
        nc.compile_mutant(control, scratch)
        res = nc.run_checks(scratch, control["checks"], control)
    finally:
        nc.revert(control, scratch)
    not_red = {k: res[k] for k in control["checks"] if res[k] != "failed"}
    assert not not_red, (f"{control['id']} ({control['desc']}): these checks did not fail on the mutant: "
                         f"{not_red}\n{res['_log']}")
