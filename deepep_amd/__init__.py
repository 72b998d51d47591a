"""deepep_amd — MI355X-native dispatch / combine / W4A8-MoE hot path behind DeepEP's interface.

``ElasticBuffer``, ``EPHandle``, ``EventHandle`` and ``EventOverlap`` keep the reference's names and
signatures (deep_ep/__init__.py:11-16).  The V1 ``Buffer`` and ``Config`` classes are outside this
build.  ``install_as_deep_ep()`` registers this package under the name ``deep_ep`` for callers that
import the reference's module path.
"""

from __future__ import annotations

import importlib
import sys

__all__ = ["ElasticBuffer", "EPHandle", "EventHandle", "EventOverlap"]

_LAZY = {
    "ElasticBuffer": ("deepep_amd.elastic", "ElasticBuffer"),
    "EPHandle": ("deepep_amd.elastic", "EPHandle"),
    "EventHandle": ("deepep_amd.event", "EventHandle"),
    "EventOverlap": ("deepep_amd.event", "EventOverlap"),
}


def __getattr__(name):
    target = _LAZY.get(name)
    if target is None:
        raise AttributeError(name)
    value = getattr(importlib.import_module(target[0]), target[1])
    globals()[name] = value
    return value


def install_as_deep_ep() -> None:
    """Make ``import deep_ep`` / ``import deep_ep_experimental.megamoe`` resolve to this package."""
    if "deep_ep" in sys.modules and sys.modules["deep_ep"] is not sys.modules[__name__]:
        raise RuntimeError("another deep_ep is already imported")
    sys.modules["deep_ep"] = sys.modules[__name__]
    sys.modules["deep_ep.utils"] = importlib.import_module("deepep_amd.utils")
    megamoe = importlib.import_module("deepep_amd.megamoe")
    experimental = type(sys)("deep_ep_experimental")
    experimental.megamoe = megamoe
    sys.modules["deep_ep_experimental"] = experimental
    sys.modules["deep_ep_experimental.megamoe"] = megamoe
