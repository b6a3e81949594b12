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
