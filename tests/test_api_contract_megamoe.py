"""Public MegaMoE signatures and argument limits match the reference's
(experiments/megamoe/python/deep_ep_experimental/megamoe/api.py, restated as data in
tests/golden/api_contract_megamoe.json; the workflow they serve is experiments/megamoe/tests/test_public_api.py:193-260)."""

import inspect
import json
import os

import pytest

from deepep_amd import megamoe
from deepep_amd.megamoe import SymmBuffer

CONTRACT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "api_contract_megamoe.json")))


def _parameters(function):
    found = []
    for parameter in inspect.signature(function).parameters.values():
        value = {"name": parameter.name, "kind": parameter.kind.name}
        if parameter.default is not inspect.Parameter.empty:
            value["default"] = list(parameter.default) if isinstance(parameter.default, tuple) else parameter.default
        found.append(value)
    return found


@pytest.mark.parametrize("name", CONTRACT["functions"])
def test_function_signature(name):
    assert _parameters(getattr(megamoe, name)) == CONTRACT["functions"][name]


@pytest.mark.parametrize("name", CONTRACT["SymmBuffer"]["methods"])
def test_buffer_method_signature(name):
    assert _parameters(getattr(SymmBuffer, name)) == CONTRACT["SymmBuffer"]["methods"][name]


def test_buffer_surface():
    public = {k for k in vars(SymmBuffer) if not k.startswith("_")}
    assert public == set(CONTRACT["SymmBuffer"]["methods"]) - {"__init__"} | set(CONTRACT["SymmBuffer"]["properties"])
    for name in CONTRACT["SymmBuffer"]["properties"]:
        assert isinstance(inspect.getattr_static(SymmBuffer, name), property)


def test_exports():
    ours = set(megamoe.__all__)
    assert ours - {"LocalGroup", "check_routing"} == set(CONTRACT["exports_reference"])


def test_argument_limits_are_the_reference_ones():
    """Every bound of api.py:93-105: the value just inside is accepted as far as validation goes (construction then
    needs a GPU, so the probe stops at the first non-ValueError), the value just outside raises ValueError."""
    limits = CONTRACT["limits"]
    base = dict(group=None, num_experts=4, num_max_tokens_per_rank=16, num_topk=2, hidden=1024, intermediate_hidden=512)

    def rejected(**change):
        try:
            SymmBuffer(**dict(base, **change)).destroy()
        except ValueError:
            return True
        except Exception:  # validation passed; torch then finds no GPU
            return False
        return False

    lo, hi = limits["hidden"]
    assert rejected(hidden=lo - limits["hidden_multiple"]) and rejected(hidden=hi + limits["hidden_multiple"])
    assert rejected(hidden=lo + limits["hidden_multiple"] // 2)
    assert not rejected(hidden=lo) and not rejected(hidden=hi) and not rejected(hidden=lo + limits["hidden_multiple"])
    lo, hi = limits["intermediate_hidden"]
    assert rejected(intermediate_hidden=lo - limits["intermediate_multiple"]) and rejected(intermediate_hidden=hi + limits["intermediate_multiple"])
    assert rejected(intermediate_hidden=lo + limits["intermediate_multiple"] // 2)
    assert not rejected(intermediate_hidden=lo) and not rejected(intermediate_hidden=hi)
    assert not rejected(intermediate_hidden=lo + limits["intermediate_multiple"])
    assert rejected(num_experts=0) and rejected(num_experts=limits["num_experts"][1] + 1)
    assert rejected(num_max_tokens_per_rank=0) and rejected(num_max_tokens_per_rank=limits["num_max_tokens_per_rank"][1] + 1)
    assert rejected(num_topk=0) and rejected(num_topk=5)  # above num_experts
    assert rejected(num_experts=64, num_topk=limits["num_topk_max"] + 1)
    assert rejected(num_shared_experts=limits["num_shared_experts"][1] + 1) and rejected(timeout=0)
    assert rejected(timeout=limits["timeout"][1] + 1)
    assert rejected(num_experts=limits["max_local_experts"] + 1)  # one rank: every expert is local
    assert not rejected(num_experts=limits["max_local_experts"])
