"""The host side of recording decode steps into graphs, without a GPU."""

from __future__ import annotations

import contextlib
import gc

import torch


def test_no_garbage_collection_while_a_step_is_recorded(monkeypatch):
    """A dropped engine's graphs may be destroyed by the collector at any allocation, and inside a
    recording that aborts the process: the recording runs with the collector off and leaves it as
    it found it, also when the step raises."""
    from tinyserve_llm_amd.engine.runner import DecodeGraphs
    inside = []

    @contextlib.contextmanager
    def fake_recording(graph, pool=None):
        inside.append(("enter", gc.isenabled(), graph, pool))
        yield
        inside.append(("exit", gc.isenabled()))

    monkeypatch.setattr(torch.cuda, "graph", fake_recording)
    assert gc.isenabled()
    assert DecodeGraphs._record("g", "p", lambda: ("ran", gc.isenabled())) == ("ran", False)
    assert inside == [("enter", False, "g", "p"), ("exit", False)] and gc.isenabled()

    def failing():
        raise RuntimeError("a kernel refused its operands")

    try:
        DecodeGraphs._record("g", None, failing)
    except RuntimeError:
        pass
    assert gc.isenabled()
    gc.disable()
    try:
        DecodeGraphs._record("g", None, lambda: None)
        assert not gc.isenabled(), "a caller that had it off keeps it off"
    finally:
        gc.enable()
