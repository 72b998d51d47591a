"""The grouped GEMM's work partition and copy/wait schedule, replayed on the host (no GPU): every span of work goes
to exactly one workgroup, and under in-order completion of vector-memory operations every asynchronous copy is
covered by a counted wait before it is read, at every tile height, tile length and launch size, with and without the
interleaved zero stores."""

import itertools

import pytest

from deepep_amd import _lib


@pytest.mark.parametrize("tile_rows", [64, 128, 192])
def test_schedule_holds_everywhere(tile_rows):
    lib = _lib.load()
    cases = 0
    for ktiles, tiles, grid, zero_blocks, epilogue in itertools.product(
        (2, 4, 6, 8, 10, 14, 16, 56, 64),                     # k = 256 ... 8192
        (0, 1, 2, 3, 5, 8, 63, 100, 192, 255, 256, 257, 288, 504, 700, 4000),
        (8, 64, 256, 304),
        (0, 3, 4, 17, 224, 5000),
        (0, 48),
    ):
        status = lib.dpep_megamoe_schedule_check(tile_rows, tiles, ktiles, grid, zero_blocks, epilogue)
        assert status == 0, (ktiles, tiles, grid, zero_blocks, epilogue, lib.dpep_last_error().decode())
        cases += 1
    assert cases > 6000


def test_schedule_check_rejects_bad_arguments():
    lib = _lib.load()
    assert lib.dpep_megamoe_schedule_check(100, 10, 8, 256, 0, 0) == -1
    assert lib.dpep_megamoe_schedule_check(128, 10, 7, 256, 0, 0) == -1
    assert b"schedule_check" in lib.dpep_last_error()
