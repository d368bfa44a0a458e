"""Tracers (pydtnn_amd/tracers.py) without a GPU: event numbering, region bookkeeping, output table."""
import pytest


class FakeLayer:
    def __init__(self, i, name):
        self.id, self.canonical_name, self.children = i, name, []
        self.canonical_name_with_id = f"{i:03}_{name}"


class FakeModel:
    def get_all_layers(self):
        return [FakeLayer(1, "Conv2D"), FakeLayer(2, "Relu")]


def test_event_numbers_are_the_reference_ones():
    from pydtnn_amd import tracers as t
    # pydtnn/tracers/events.py:25-70
    assert (t.PYDTNN_MDL_EVENT, t.PYDTNN_MDL_EVENTS, t.PYDTNN_OPS_EVENT, t.PYDTNN_OPS_EVENTS) == \
        (60000001, 5, 60000002, 36)
    assert (t.PYDTNN_MDL_FORWARD, t.PYDTNN_MDL_BACKWARD, t.PYDTNN_MDL_UPDATE_DW) == (1, 2, 5)
    assert t.PYDTNN_OPS_ALLREDUCE_DW == 1 and t.PYDTNN_OPS_BACKWARD_CONVGEMM == 2
    assert t.PYDTNN_OPS_BACKWARD_DECONV_GEMM == 9 and t.PYDTNN_OPS_COMP_DW_MATMUL == 18
    assert t.PYDTNN_OPS_FORWARD_CONVGEMM == 24 and t.PYDTNN_OPS_FORWARD_IM2COL == 30
    assert t.PYDTNN_OPS_FORWARD_MATMUL == 31 and t.PYDTNN_OPS_FORWARD_TRANSPOSE_Y == 36


def test_simple_tracer_times_nested_regions_and_writes_the_table(tmp_path, monkeypatch):
    from pydtnn_amd import tracers as t
    now = [0.0]
    monkeypatch.setattr(t, "timer", lambda: now[0])
    out = tmp_path / "trace.csv"
    tr = t.SimpleTracer(True, str(out), sync=lambda: None)
    tr.define_event_types(FakeModel())
    fwd = 1 * t.PYDTNN_MDL_EVENTS + t.PYDTNN_MDL_FORWARD
    op = 1 * t.PYDTNN_OPS_EVENTS + t.PYDTNN_OPS_FORWARD_CONVGEMM
    for _ in range(3):
        tr.emit_event(t.PYDTNN_MDL_EVENT, fwd)
        now[0] += 1.0
        tr.emit_event(t.PYDTNN_OPS_EVENT, op)
        now[0] += 2.0
        tr.emit_event(t.PYDTNN_OPS_EVENT, 0)
        tr.emit_event(t.PYDTNN_MDL_EVENT, 0)
    tr.emit_nevent([t.PYDTNN_MDL_EVENT, t.PYDTNN_OPS_EVENT], [fwd, op])
    now[0] += 4.0
    tr.emit_nevent([t.PYDTNN_MDL_EVENT, t.PYDTNN_OPS_EVENT], [0, 0])
    assert tr.events[t.PYDTNN_OPS_EVENT][op] == [4, [2.0, 2.0, 2.0, 4.0]]
    assert tr.events[t.PYDTNN_MDL_EVENT][fwd] == [4, [3.0, 3.0, 3.0, 4.0]]
    with pytest.raises(ValueError):
        tr.emit_event(t.PYDTNN_OPS_EVENT, 0)                      # nothing open
    tr.emit_event(t.PYDTNN_MDL_EVENT, fwd)
    with pytest.raises(ValueError):
        tr.emit_event(t.PYDTNN_OPS_EVENT, 0)                      # closes the wrong type
    assert tr.events[t.PYDTNN_OPS_EVENT][12345] == [0, []]       # a lookup leaves an entry without durations behind
    tr.write_output()                                             # ... which the table skips
    lines = out.read_text().splitlines()
    assert lines[0] == "Event type;Event value;Event name;Calls;Total time;Median of times"
    assert f"Operations;{op};001_Conv2D_forward_convgemm;4;10.0;2.0" in lines
    assert f"Model;{fwd};001_Conv2D_forward;4;13.0;3.0" in lines


def test_disabled_tracer_records_nothing():
    from pydtnn_amd import tracers as t
    tr = t.SimpleTracer(False, "unused.csv", sync=lambda: None)
    tr.emit_event(t.PYDTNN_MDL_EVENT, 6)
    tr.emit_event(t.PYDTNN_MDL_EVENT, 0)
    assert not tr.events and not tr.pending_events
    t.NullTracer().emit_nevent([1], [2])
