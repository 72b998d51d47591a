"""The grouped GEMM's copy/wait schedule, replayed on the host (no GPU): under in-order completion of vector-memory
operations every asynchronous copy is covered by a counted wait before it is read (an item's operands before its
MFMAs, the next tile's gather indices before the copy cursor switches tiles), at every tile height, k length and
number of tiles per workgroup.  The short-k corner matters: with four k tiles (k = 512) a tile is shorter than the ring
of the 64- and 128-row kernels, and the cursor has to let everything land before it reads the next tile's indices."""

import itertools

import pytest

from deepep_amd import _lib


@pytest.mark.parametrize("tile_rows", [64, 128, 192])
def test_schedule_holds_everywhere(tile_rows):
    lib = _lib.load()
    cases = 0
    for ktiles, tiles, epilogue in itertools.product((2, 4, 6, 8, 10, 14, 16, 56, 64), (0, 1, 2, 3, 5, 24, 100), (0, 48, 192)):
        status = lib.dpep_megamoe_schedule_check(tile_rows, tiles, ktiles, epilogue, 0)
        assert status == 0, (ktiles, tiles, epilogue, lib.dpep_last_error().decode())
        cases += 1
    assert cases == 9 * 7 * 3


def test_schedule_check_rejects_bad_arguments():
    lib = _lib.load()
    assert lib.dpep_megamoe_schedule_check(100, 10, 8, 0, 0) == -1
    assert lib.dpep_megamoe_schedule_check(128, 10, 7, 0, 0) == -1
    assert b"schedule_check" in lib.dpep_last_error()


@pytest.mark.parametrize("tile_rows,ahead", [(64, 5), (128, 4), (192, 3)])
def test_replay_catches_a_schedule_without_the_wait_at_switches(tile_rows, ahead):
    """The same replay with the cursor's wait at tile switches left out fails exactly where the rule says the wait is
    needed: more than one tile per workgroup and either a switch inside the prologue (tiles no longer than the copies
    run ahead) or tiles shorter than that.  Long tiles pass either way: a counted wait has covered the index fetch."""
    lib = _lib.load()
    for ktiles, tiles in itertools.product((2, 4, 6, 8, 16, 56), (1, 2, 3, 24)):
        status = lib.dpep_megamoe_schedule_check(tile_rows, tiles, ktiles, 48, 1)
        must_fail = tiles > 1 and ktiles <= ahead
        assert (status != 0) == must_fail, (tile_rows, ktiles, tiles, lib.dpep_last_error().decode())
        if must_fail:
            assert b"gather indices" in lib.dpep_last_error()


@pytest.mark.parametrize("tile_rows", [64, 128, 192])
def test_column_wave_schedule_holds_everywhere(tile_rows):
    """The kernel that runs where K is a multiple of 512: every item's activation copies and weight loads, and every
    tile's gather indices, are covered by a counted wait at every k length (in fours) and number of tiles."""
    lib = _lib.load()
    for ktiles, tiles, epilogue in itertools.product((4, 8, 12, 16, 56, 64), (0, 1, 2, 3, 5, 24, 100), (0, 12, 96)):
        status = lib.dpep_megamoe_schedule_check_column_waves(tile_rows, tiles, ktiles, epilogue, 0)
        assert status == 0, (ktiles, tiles, epilogue, lib.dpep_last_error().decode())
    assert lib.dpep_megamoe_schedule_check_column_waves(tile_rows, 3, 6, 0, 0) == -1  # k tiles come in fours
    assert lib.dpep_megamoe_schedule_check_column_waves(96, 3, 8, 0, 0) == -1


@pytest.mark.parametrize("tile_rows,requests", [(64, 6), (128, 8), (192, 10)])
def test_column_wave_replay_catches_a_wait_that_is_too_lax(tile_rows, requests):
    """One more item's requests allowed in flight than the kernel allows: the next item's operands are then not
    guaranteed, and the replay says so.  A few operations of slack are absorbed only where a span's or a tile's extra
    copies sit between the items (the real count ignores those, which errs on the strict side)."""
    lib = _lib.load()
    for ktiles, tiles in itertools.product((4, 8, 16, 56), (1, 2, 24)):
        assert lib.dpep_megamoe_schedule_check_column_waves(tile_rows, tiles, ktiles, 12, requests) == -1, (ktiles, tiles)
        assert b"operands" in lib.dpep_last_error()
        assert lib.dpep_megamoe_schedule_check_column_waves(tile_rows, tiles, ktiles, 12, 0) == 0


@pytest.mark.parametrize("tile_rows,ahead", [(64, 5), (128, 4), (192, 3)])
def test_replay_catches_scale_slots_reused_too_early(tile_rows, ahead):
    """The scales of a span of k tiles sit in a ring of LDS slots; the replay also checks that a slot is refilled only
    when the span it held has been read to the end.  With the two slots the 2 x 2 kernel used to have, a tile whose k is no
    multiple of 512 (a last span of two k tiles) breaks that in a workgroup with more than one tile wherever the copies run
    more than three items ahead (64- and 128-row tiles); with three slots, and with whole spans, it holds everywhere."""
    lib = _lib.load()
    two_slots = 2
    for ktiles, tiles in itertools.product((4, 6, 8, 10, 14, 16, 18), (1, 2, 3, 24)):
        assert lib.dpep_megamoe_schedule_check(tile_rows, tiles, ktiles, 48, 0) == 0, (ktiles, tiles, lib.dpep_last_error().decode())
        status = lib.dpep_megamoe_schedule_check(tile_rows, tiles, ktiles, 48, two_slots)
        must_fail = tiles > 1 and ktiles % 4 == 2 and ahead > 3
        assert (status != 0) == must_fail, (tile_rows, ktiles, tiles, lib.dpep_last_error().decode())
        if must_fail:
            assert b"overwritten" in lib.dpep_last_error()
