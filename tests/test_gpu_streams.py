"""Stream order of ElasticBuffer calls under a seeded random schedule: inputs produced late (behind a sleeping kernel) on
one of three streams, synchronous calls on the caller's stream and asynchronous ones on the communication stream mixed
freely, `previous_event` given or not, results consumed on yet another stream after waiting for the returned event.
Every iteration's dispatch and combine are compared with the CPU oracle bit for bit: a missing dependency between two
streams shows as rows read before their producer ran."""

import numpy as np
import pytest
import torch

from oracle import combine as ocombine
from oracle import layout as olayout
from tests.gpu_util import bf16_bits

pytestmark = pytest.mark.gpu

SLEEP_CYCLES = 3_000_000  # about 1.5 ms: far longer than the host needs to queue the next call


@pytest.mark.parametrize("world,seed", [(1, 0), (4, 1)])  # world 1: outputs allocated before R is known; world 4: after
def test_calls_wait_for_their_producers_whatever_the_streams(world, seed):
    import deepep_amd
    from deepep_amd.event import EventHandle

    tokens, hidden, topk, experts = 96, 512, 4, 16
    rng = np.random.default_rng(seed)
    torch.cuda.set_device(0)
    streams = [torch.cuda.current_stream(), torch.cuda.Stream(), torch.cuda.Stream()]
    buffer = deepep_amd.ElasticBuffer(None, num_max_tokens_per_rank=tokens, hidden=hidden, num_topk=topk, rank=world - 1,
                                      world_size=world, explicitly_destroy=True)
    per_rank = experts // world
    try:
        for it in range(20):
            case = dict(world=world, seed=seed, it=it)
            ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64)
            ids[rng.random(ids.shape) < 0.15] = -1
            x_host = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32)).bfloat16()
            want = olayout.layout(ids, experts, (world - 1) * per_rank, per_rank)
            rows = want["num_rows"]
            y_host = torch.from_numpy(rng.normal(size=(rows, hidden)).astype(np.float32)).bfloat16()
            produce_on, consume_on = streams[rng.integers(0, 3)], streams[rng.integers(0, 3)]
            dispatch_async, combine_async = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
            staged_x, staged_y, idx = x_host.cuda(), y_host.cuda(), torch.from_numpy(ids).cuda()
            torch.cuda.synchronize()
            with torch.cuda.stream(produce_on):
                torch.cuda._sleep(SLEEP_CYCLES)
                x = staged_x * 1  # exists only once the sleep is over
                after_x = EventHandle()
            call_on = streams[rng.integers(0, 3)]
            with torch.cuda.stream(call_on):
                # a call on another stream than the producer's needs the producer's event; on the same stream the order is the stream's
                previous = after_x if (call_on is not produce_on or rng.integers(0, 2)) else None
                recv, _, _, handle, event = buffer.dispatch(x, topk_idx=idx, num_experts=experts, previous_event=previous,
                                                            async_with_compute_stream=dispatch_async)
                if dispatch_async:
                    event.current_stream_wait()
                assert handle.num_expanded_tokens == rows, case
                got_rows = bf16_bits(recv)  # (the copy to the host runs on call_on, behind the event)
                np.testing.assert_array_equal(got_rows, olayout.expand_rows(bf16_bits(x_host), want["row_to_route"], topk), err_msg=str(case))
            with torch.cuda.stream(produce_on):
                torch.cuda._sleep(SLEEP_CYCLES)
                y = staged_y * 1
                after_y = EventHandle()
            with torch.cuda.stream(call_on):
                previous = after_y if (call_on is not produce_on or rng.integers(0, 2)) else None
                out, _, event = buffer.combine(y, handle, previous_event=previous, async_with_compute_stream=combine_async)
                done = EventHandle() if not combine_async else None
            with torch.cuda.stream(consume_on):
                if combine_async:
                    event.current_stream_wait()
                else:
                    done.current_stream_wait()
                doubled = out.float() * 2  # a consumer kernel on the third stream
                np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(y_host), want["route_to_row"]), err_msg=str(case))
                assert torch.equal(doubled, out.float() * 2)
            torch.cuda.synchronize()
        assert not buffer._runtime.notify_failed
    finally:
        torch.cuda.synchronize()
        buffer.destroy()


def test_mega_moe_calls_on_alternating_streams_share_the_workspace_in_order():
    """Two forwards of one SymmBuffer queued on different streams, the first behind a sleeping kernel: the second has to
    wait for the first (they share the workspace), and each has to produce its own inputs' result."""
    from deepep_amd import megamoe
    from oracle import megamoe as mm
    from tests.test_gpu_megamoe import _make_problem, _oracle

    tokens, hidden, inter, experts, topk = 200, 1024, 512, 8, 2
    problems = [_make_problem(tokens, hidden, inter, experts, 0, experts, topk, seed=s) for s in (21, 22)]
    l1, l2 = problems[0][2], problems[0][3]  # one set of weights, two batches
    buf = megamoe.SymmBuffer(None, experts, tokens, topk, hidden, inter)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    try:
        p1, p2 = megamoe.transform_weights_for_mega_moe(
            (torch.from_numpy(l1[0]).cuda(), torch.from_numpy(l1[1]).cuda()), (torch.from_numpy(l2[0]).cuda(), torch.from_numpy(l2[1]).cuda()))
        staged = [(torch.from_numpy(pr[0]).cuda().view(torch.float8_e4m3fn), torch.from_numpy(pr[1]).cuda(), torch.from_numpy(pr[4]).cuda(),
                   torch.from_numpy(pr[5]).cuda()) for pr in problems]
        torch.cuda.synchronize()
        for round_ in range(4):
            outs = []
            for which, stream in enumerate(streams if round_ % 2 == 0 else streams[::-1]):
                codes, scales, ids, wts = staged[which]
                with torch.cuda.stream(stream):
                    if which == 0:
                        torch.cuda._sleep(SLEEP_CYCLES)
                    y, counts = megamoe.mega_moe((codes, scales), ids, wts, p1, p2, buf)
                    outs.append((which, y, counts))
            torch.cuda.synchronize()
            for which, y, counts in outs:
                x_codes, x_scales, _, _, idx, weights = problems[which]
                assert counts.cpu().tolist() == np.bincount(idx.ravel(), minlength=experts).tolist(), (round_, which)
                want = _oracle(x_codes, x_scales, l1, l2, idx, weights, 0)
                err = mm.relative_frobenius(y.float().cpu().numpy(), want)
                assert err <= 2e-2, (round_, which, err)
    finally:
        torch.cuda.synchronize()
        buf.destroy()


def test_two_threads_with_buffers_of_their_own():
    """Two host threads, each with its own ElasticBuffer and stream, dispatching and combining at the same time: the
    library keeps no state that one thread's calls could take from the other's (the error text is per thread, workspaces
    are per buffer), so each thread's results are its own inputs' results."""
    import threading

    import deepep_amd

    tokens, hidden, topk, experts = 300, 1024, 4, 32
    failures = []

    def work(seed):
        try:
            torch.cuda.set_device(0)
            rng = np.random.default_rng(seed)
            stream = torch.cuda.Stream()
            buffer = deepep_amd.ElasticBuffer(None, num_max_tokens_per_rank=tokens, hidden=hidden, num_topk=topk, explicitly_destroy=True)
            try:
                with torch.cuda.stream(stream):
                    for it in range(12):
                        ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64)
                        ids[rng.random(ids.shape) < 0.1] = -1
                        x = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32)).bfloat16()
                        recv, _, _, handle, _ = buffer.dispatch(x.cuda(), topk_idx=torch.from_numpy(ids).cuda(), num_experts=experts)
                        want = olayout.layout(ids, experts)
                        np.testing.assert_array_equal(bf16_bits(recv), olayout.expand_rows(bf16_bits(x), want["row_to_route"], topk))
                        out, _, _ = buffer.combine(recv, handle)
                        np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(recv), want["route_to_row"]))
                        with pytest.raises(ValueError, match="hidden differs"):  # this thread's error, with this thread's text
                            buffer.dispatch(x[:, :512].contiguous().cuda(), topk_idx=torch.from_numpy(ids).cuda(), num_experts=experts)
            finally:
                torch.cuda.synchronize()
                buffer.destroy()
        except BaseException as error:  # noqa: BLE001 - reported by the main thread
            failures.append((seed, repr(error)))

    threads = [threading.Thread(target=work, args=(seed,)) for seed in (1, 2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert not failures, failures
