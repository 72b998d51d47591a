"""Keyword spelling policy of the public API.

Published signatures keep the upstream DeepEP spellings (``num_sms``, ``num_gpu_timeout_secs``,
``use_tma_aligned_col_major_sf``); the Ascend project's spellings (``num_compute_units``,
``num_device_timeout_secs``, ``use_aligned_col_major_sf``) stay accepted as aliases, as in the
reference (deep_ep/_compat.py:52-72, applied in deep_ep/backends/mesh_clos/elastic.py:1536-1556).
Values are never rescaled; passing both spellings with different values is a TypeError.
"""

from __future__ import annotations

import functools


def accept_aliases(**alias_to_public):
    """Decorator: ``alias=value`` is forwarded as ``public=value``; the signature is unchanged."""

    def wrap(function):
        @functools.wraps(function)
        def call(*args, **kwargs):
            for alias, public in alias_to_public.items():
                if alias in kwargs:
                    value = kwargs.pop(alias)
                    if public in kwargs and kwargs[public] != value:
                        raise TypeError(f"conflicting {alias} and {public}")
                    kwargs[public] = value
            return function(*args, **kwargs)

        return call

    return wrap
