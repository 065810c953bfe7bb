"""CPU: which split-group workspaces a schedule keeps, hands out under graph capture and gives back.

A captured graph holds the raw address of its workspace, so a buffer handed out under capture must
never return to the allocator; an eager one may, once the stream it was used on has drained."""
import pytest
import torch


@pytest.fixture
def sched(monkeypatch):
    from sparse import _ops
    s = _ops.Schedule.__new__(_ops.Schedule)
    s.table = torch.empty(1)                      # a CPU tensor: torch.zeros(device=...) below stays on the host
    s._workspaces, s._captured, s._spares, s.last_key = {}, {}, {}, None
    s.drained = []
    monkeypatch.setattr(s, "_drain", lambda handle: s.drained.append(handle))
    state = {"capturing": False}
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: state["capturing"])
    s.state = state
    return s


def test_eager_buffers_are_reused_and_zero(sched):
    a, n = sched._zeroed(("dsd", 4, 64, 64, 7), 256)
    assert n == 256 and a.numel() == 256 and int(a.sum()) == 0
    b, _ = sched._zeroed(("dsd", 4, 64, 64, 7), 256)
    assert b.data_ptr() == a.data_ptr()
    c, _ = sched._zeroed(("dsd", 4, 64, 64, 9), 256)          # another stream: its own buffer
    assert c.data_ptr() != a.data_ptr()
    assert sched._zeroed(("dsd", 4, 64, 64, 7), 0) == (None, 0)


def test_capture_takes_the_spare_and_never_gives_it_back(sched):
    key = ("dds", 16, 64, 4096, 3)
    sched.state["capturing"] = True
    with pytest.raises(RuntimeError):                           # never run eagerly: nothing zeroed is at hand
        sched._zeroed(key, 128)
    sched.state["capturing"] = False
    eager, _ = sched._zeroed(key, 128)                          # leaves a zeroed spare for this shape
    other_stream = key[:-1] + (5,)
    sched.state["capturing"] = True
    captured, _ = sched._zeroed(other_stream, 128)
    assert captured.data_ptr() != eager.data_ptr() and int(captured.sum()) == 0
    again, _ = sched._zeroed(other_stream, 128)                 # the same graph asks again: the same buffer
    assert again.data_ptr() == captured.data_ptr()
    sched.state["capturing"] = False
    # a flood of eager shapes evicts eager buffers only
    for i in range(3 * sched.MAX_WORKSPACES):
        sched._zeroed(("dsd", i + 1, 64, 64, 11), 64)
    assert len(sched._workspaces) == sched.MAX_WORKSPACES
    assert other_stream in sched._captured and sched._captured[other_stream].data_ptr() == captured.data_ptr()
    assert key not in sched._workspaces                         # the oldest eager one went ...
    assert sched.drained and sched.drained[0] == key[-1]        # ... after its stream was waited for
    assert len(sched.drained) == 1 + 3 * sched.MAX_WORKSPACES - sched.MAX_WORKSPACES


def test_an_eager_buffer_moves_to_the_graph_that_captures_it(sched):
    key = ("dsd", 2, 64, 64, 1)
    eager, _ = sched._zeroed(key, 64)
    sched.state["capturing"] = True
    captured, _ = sched._zeroed(key, 64)
    assert captured.data_ptr() == eager.data_ptr()
    assert key in sched._captured and key not in sched._workspaces
    sched.state["capturing"] = False
    later, _ = sched._zeroed(key, 64)                           # eager calls on that stream keep using it
    assert later.data_ptr() == eager.data_ptr()
    sched.discard(key)                                          # a failed launch: forget it wherever it is
    assert key not in sched._captured and key not in sched._workspaces
