"""The negative-control table itself (no GPU): every control's text occurs exactly once in its file,
the mutated file differs, a stale control is an error, and the checks it names exist."""
import os
import subprocess
import sys

import pytest

import negative_controls as nc
import util


@pytest.fixture(scope="module")
def scratch(tmp_path_factory):
    return nc.make_scratch(str(tmp_path_factory.mktemp("negctl") / "tree"))


def test_every_control_applies_exactly_once_and_is_taken_back(scratch):
    controls = nc.read_table()
    assert len(controls) >= 10 and len({c["id"] for c in controls}) == len(controls)
    for c in controls:
        real = open(os.path.join(util.ROOT, c["file"])).read()
        path = nc.apply(c, scratch)
        assert open(path).read() != real, c["id"]
        nc.revert(c, scratch)
        assert open(path).read() == real, c["id"]


def test_a_control_whose_text_has_moved_on_is_an_error(scratch):
    c = dict(nc.read_table()[0], old="this text is nowhere in the file")
    with pytest.raises(nc.StaleControl, match="occurs 0 times"):
        nc.apply(c, scratch)
    twice = dict(c, old="const int")
    with pytest.raises(nc.StaleControl, match="not once"):
        nc.apply(twice, scratch)


def test_the_checks_named_in_the_table_exist():
    checks = sorted({k for c in nc.read_table() for k in c["checks"]})
    p = subprocess.run([sys.executable, "-m", "pytest", "--collect-only", "-q", "-p", "no:cacheprovider", *checks],
                       cwd=util.ROOT, capture_output=True, text=True)
    listed = set(p.stdout.split())
    assert p.returncode == 0 and all(k in listed for k in checks), [k for k in checks if k not in listed]


def test_the_scratch_copy_holds_sources_only(scratch):
    for folder, dirs, files in os.walk(scratch, followlinks=False):
        assert not [f for f in files if f.endswith((".so", ".pyc"))], folder
    assert os.path.islink(os.path.join(scratch, "tuff_amd", "csrc", "_lib")) or \
        not os.path.isdir(os.path.join(util.ROOT, "tuff_amd", "csrc", "_lib"))


def test_the_frozen_vectors_are_well_formed():
    """tests/golden/*.json: one file a configuration, a sha256 and a first choice for every row of every fixed
    request, the fingerprint of the environment that made them, and the configurations that were byte-identical."""
    import json
    import golden
    for name in golden.NAMES:
        with open(golden.path_of(name)) as f:
            g = json.load(f)
        assert g["format"] == golden.FORMAT and g["configuration"] == name and g["dtype"] == "float32"
        reqs = golden.requests_for(name)
        assert set(g["requests"]) == set(reqs)
        for rid, toks in reqs.items():
            r = g["requests"][rid]
            assert r["tokens"] == len(toks) == len(r["row_sha256"]) == len(r["top1"])
            assert all(len(h) == 64 and int(h, 16) >= 0 for h in r["row_sha256"])
        assert set(g["environment"]["fingerprint"]) == {"gpu_arch", "hipcc"}
        assert len(g["provenance"]["configurations_verified_identical"]) == len(golden.configurations()) and g["provenance"]["reason"]
        assert len(g["model"]["safetensors_sha256"]) == 64
