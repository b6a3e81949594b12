"""Host logic of the side stream's numbered work (conef_amd._pools.side_recorded / side_wait):
which waits are issued and which are covered by an earlier one.  No GPU: streams and events are
stand-ins that note what they are asked to do."""
import torch

from conef_amd import _pools


class FakeStream:
    def __init__(self, handle):
        self.cuda_stream = handle
        self.waited_for = []

    def wait_event(self, event):
        self.waited_for.append(event)


def test_one_wait_covers_everything_recorded_before_it():
    device = torch.device("cpu")
    _pools._SIDE_ORDER.pop(device, None)
    try:
        events = ["e%d" % i for i in range(6)]
        numbers = [_pools.side_recorded(device, e) for e in events[:4]]
        assert numbers == [1, 2, 3, 4]
        main = FakeStream(11)
        # the oldest piece of work is asked for first: the wait goes to the newest event ...
        _pools.side_wait(device, main, numbers[0])
        assert main.waited_for == ["e3"]
        # ... and covers the rest of what had been recorded by then
        for n in numbers[1:]:
            _pools.side_wait(device, main, n)
        assert main.waited_for == ["e3"]
        # work recorded afterwards needs a wait of its own, again on the newest event
        later = [_pools.side_recorded(device, e) for e in events[4:]]
        _pools.side_wait(device, main, later[0])
        assert main.waited_for == ["e3", "e5"]
        _pools.side_wait(device, main, later[1])
        assert main.waited_for == ["e3", "e5"]
        # another stream has waited for nothing yet
        other = FakeStream(12)
        _pools.side_wait(device, other, numbers[1])
        assert other.waited_for == ["e5"]
        # nothing to wait for
        _pools.side_wait(device, other, None)
        assert other.waited_for == ["e5"]
    finally:
        _pools._SIDE_ORDER.pop(device, None)


def test_release_forgets_the_numbering():
    device = torch.device("cpu")
    _pools._SIDE_ORDER.pop(device, None)
    number = _pools.side_recorded(device, "e")
    _pools.release()                    # waits for the devices it knows and drops every pool
    assert device not in _pools._SIDE_ORDER
    stream = FakeStream(5)
    _pools.side_wait(device, stream, number)      # the device was idle when the pools were dropped
    assert stream.waited_for == []


def test_a_rebuilt_round_plan_still_waits_for_the_side_stream():
    """The error tensors and the Q arena of a bucket outlive its round plan, which is replaced
    whenever the bucket's buffer moves: the top-k the replaced plan left on the side stream must
    still be waited for by the next round, and so must its copy of the Q arena."""
    from types import SimpleNamespace

    from conef_amd import _psgd_engine as engine

    device = torch.device("cpu")
    _pools._SIDE_ORDER.pop(device, None)
    try:
        state = SimpleNamespace(round_cache={}, matrix_approximation_rank=2, min_compression_rate=2)
        grads = [torch.zeros(16, 32), torch.zeros(7)]
        main = FakeStream(21)
        first = engine.plan_for(state, 0, grads, ("buffer-a",), "topk", device, lambda: main)
        assert state.round_cache[0] is first and first.count == 1 and main.waited_for == []
        # the same key: the same plan, nothing to order
        assert engine.plan_for(state, 0, grads, ("buffer-a",), "topk", device, lambda: main) is first
        # the same buffer with another layout: a new plan
        assert engine.plan_for(state, 0, grads[:1], ("buffer-a",), "topk", device, lambda: main) is not first
        first = engine.plan_for(state, 0, grads, ("buffer-a",), "topk", device, lambda: main)
        # its round left a top-k and a Gram-Schmidt of the next Q factors on the side stream
        first.topk_event = "topk-done"
        first.topk_number = _pools.side_recorded(device, "topk-done")
        # the bucket's buffer moves: a new plan, which inherits the pending top-k ...
        second = engine.plan_for(state, 0, grads, ("buffer-b",), "topk", device, lambda: main)
        assert second is not first and state.round_cache[0] is second
        assert (second.topk_number, second.topk_event) == (first.topk_number, "topk-done")
        assert main.waited_for == []
        # ... and its round waits for it before it touches the error tensors, once
        engine.wait_for_side_topk(second, device, lambda: main)
        assert main.waited_for == ["topk-done"] and second.topk_number is None
        engine.wait_for_side_topk(second, device, lambda: main)
        assert main.waited_for == ["topk-done"]
        # settle() (state_dict, clean_error) still finds the event through the new plan
        assert [p.topk_event for p in state.round_cache.values()] == ["topk-done"]
        # a pending copy of the Q arena is waited for when the plan that knew of it goes
        second.q_next_number = _pools.side_recorded(device, "q-copied")
        third = engine.plan_for(state, 0, grads, ("buffer-c",), "topk", device, lambda: main)
        assert third.q_next_number is None and main.waited_for == ["topk-done", "q-copied"]
    finally:
        _pools._SIDE_ORDER.pop(device, None)


def test_a_stale_topk_table_is_told_from_a_current_one():
    from conef_amd import _psgd_engine as engine
    tensors = [torch.zeros(8), torch.zeros(9)]
    key = tuple(t.data_ptr() for t in tensors)
    table = (key, None, None, None, None, 0.4)
    assert engine.topk_table_is_stale(None, tensors, 0.4)
    assert not engine.topk_table_is_stale(table, tensors, 0.4)
    assert engine.topk_table_is_stale(table, tensors, 0.3)                         # another ratio
    assert engine.topk_table_is_stale(table, [tensors[0], torch.zeros(9)], 0.4)    # an error tensor was replaced
