"""Public signatures match the reference's machine-readable contract (tests/api/api_contract.json,
checked there by tests/api/test_contracts.py:52-69), for the classes this build provides."""

import copy
import inspect
import json
import os

import pytest

import deepep_amd

CONTRACT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "api_contract_elastic.json")))
METHODS = [(n, m, s) for n, o in CONTRACT["objects"].items() for m, s in o["methods"].items()]


@pytest.mark.parametrize("name,method,spec", METHODS, ids=[f"{n}.{m}" for n, m, _ in METHODS])
def test_signature_matches_contract(name, method, spec):
    expected = copy.deepcopy(spec["parameters"])
    for deviation in CONTRACT["deviations"]:
        if deviation["symbol"] == f"{name}.{method}":
            parameter = next(p for p in expected if p["name"] == deviation["parameter"])
            parameter["default"] = deviation["project_default"]
    cls = getattr(deepep_amd, name)
    actual = []
    for parameter in inspect.signature(getattr(cls, method)).parameters.values():
        value = {"name": parameter.name, "kind": parameter.kind.name}
        if parameter.default is not inspect.Parameter.empty:
            value["default"] = parameter.default
        actual.append(value)
    assert actual == expected
    assert isinstance(inspect.getattr_static(cls, method), staticmethod) == (spec["kind"] == "staticmethod")


@pytest.mark.parametrize("name", CONTRACT["objects"])
def test_no_undeclared_public_methods(name):
    cls = getattr(deepep_amd, name)
    public = {k for k, v in inspect.getmembers(cls) if not k.startswith("_") and (callable(v) or isinstance(v, staticmethod))}
    assert public == {k for k in CONTRACT["objects"][name]["methods"] if not k.startswith("_")}


def test_exports():
    assert set(deepep_amd.__all__) == {"ElasticBuffer", "EPHandle", "EventHandle", "EventOverlap"}
