"""CPU restatement of the reference's dispatch / combine / MegaMoE semantics.

TEST INFRASTRUCTURE ONLY.  Nothing under ``deepep_amd/`` imports this package:
it is the checker used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.  The product path is the HIP library and
fails loudly when that library is missing.

Every function cites the reference file:line it restates (paths relative to the
reference checkout).  Pinning status (which reference-held vector or
mathematical identity fixes each function) is listed per module; a function
that nothing pins says "parity unpinned" in its docstring.
"""

from . import layout, quant, combine, megamoe, cases  # noqa: F401
