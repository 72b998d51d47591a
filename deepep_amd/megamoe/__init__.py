"""W4A8 MegaMoE forward with the reference's experimental interface
(experiments/megamoe/python/deep_ep_experimental/megamoe/api.py)."""

from .api import (  # noqa: F401
    LocalGroup,
    StoreGroup,
    SymmBuffer,
    fp8_fp4_mega_moe,
    mega_moe,
    transform_weights_for_mega_moe,
)
from .validation import check_routing  # noqa: F401

__all__ = ["LocalGroup", "StoreGroup", "SymmBuffer", "transform_weights_for_mega_moe", "mega_moe", "fp8_fp4_mega_moe", "check_routing"]
