"""MegaMoE host-side checks that need no GPU: argument gates and the routing preflight
(experiments/megamoe/tests/test_public_api.py:233-238, validation.py:10-22)."""

import pytest

from deepep_amd.megamoe import LocalGroup, SymmBuffer, check_routing


def test_check_routing_messages():
    check_routing([[0, 1], [2, 3]], [[0.5, 0.5], [0.1, 0.9]], 4, 2)
    for bad in (-1, 4, 1):
        with pytest.raises(ValueError, match=r"rank=0.*token=0"):
            check_routing([[bad, 1]], [[0.5, 0.5]], 4, 2)
    with pytest.raises(ValueError, match="finite"):
        check_routing([[0, 1]], [[float("nan"), 0.5]], 4, 2)
    with pytest.raises(ValueError, match="top-k"):
        check_routing([[0]], [[0.5]], 4, 2)
    with pytest.raises(ValueError, match="rank=3"):
        check_routing([[0, 0]], [[0.5, 0.5]], 4, 2, rank=3)


def test_symm_buffer_argument_gates():
    for kwargs in (
        dict(num_experts=0), dict(num_topk=0), dict(hidden=512), dict(hidden=1024 + 32), dict(intermediate_hidden=128), dict(intermediate_hidden=320),
        dict(num_topk=5), dict(num_experts=6, group=LocalGroup(0, 4)),
    ):
        args = dict(group=None, num_experts=4, num_max_tokens_per_rank=17, num_topk=2, hidden=1024, intermediate_hidden=512)
        args.update(kwargs)
        with pytest.raises(ValueError):
            SymmBuffer(**args)
    with pytest.raises(ValueError):
        SymmBuffer(None, 4, 17, 2, 1024, 512, num_shared_experts=9)
    with pytest.raises(TypeError):
        SymmBuffer(object(), 4, 17, 2, 1024, 512)
    with pytest.raises(ValueError):
        LocalGroup(2, 2)


def test_store_group_is_the_launchers_identity(monkeypatch):
    """StoreGroup.from_env() as the reference's example calls it (README.md:247): rank and size from the launcher's
    environment, no store behind it; the coordinating calls answer for this process."""
    from deepep_amd.megamoe import StoreGroup

    monkeypatch.delenv("RANK", raising=False)
    monkeypatch.delenv("WORLD_SIZE", raising=False)
    alone = StoreGroup.from_env()
    assert (alone.rank(), alone.size()) == (0, 1) and isinstance(alone, LocalGroup)
    assert alone.barrier("before SHMEM teardown") is None and alone.all_gather({"rows": 3}, "sizes") == [{"rows": 3}]
    assert alone.abort("MegaMoE: RuntimeError: x") is None and alone.close() is None
    monkeypatch.setenv("RANK", "5")
    monkeypatch.setenv("WORLD_SIZE", "8")
    share = StoreGroup.from_env(timeout=30)
    assert (share.rank(), share.size()) == (5, 8)
    with pytest.raises(NotImplementedError, match="transport"):
        share.all_gather(1, "x")
    with pytest.raises(ValueError):
        StoreGroup.from_env(timeout=0)
