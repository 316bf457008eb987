"""The committed digests of the five benchmark configurations
(tests/golden/config_fixtures.json) against what the input generators and the
CPU oracle produce today: a drift of numpy's Philox streams, of the generators
or of the oracle fails here, on the CPU, before any GPU comparison."""
import importlib.util
import json
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = json.load(open(os.path.join(HERE, "golden", "config_fixtures.json")))

_spec = importlib.util.spec_from_file_location("make_config_fixtures",
                                               os.path.join(HERE, "golden", "make_config_fixtures.py"))
make = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make)


@pytest.mark.parametrize("name,fn", [("configs[0]", "config1"), ("configs[1]", "config2"), ("configs[2]", "config3"),
                                     ("configs[3]", "config4"), ("configs[4]", "config5")])
def test_generators_and_oracle_reproduce_the_committed_digests(name, fn):
    assert getattr(make, fn)() == FIXTURES[name]


def test_fixture_file_is_complete():
    assert set(FIXTURES) >= {f"configs[{i}]" for i in range(5)}
    assert FIXTURES["configs[1]"]["x"]["shape"] == [16384, 16384]
    assert FIXTURES["configs[2]"]["y"]["shape"] == [4096, 4096]
    assert set(FIXTURES["configs[3]"]) >= {"M=1", "M=8", "M=32", "M=128"}
    assert FIXTURES["configs[4]"]["layer2"]["y"]["shape"] == [256, 1024]
