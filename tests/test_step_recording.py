"""What the step function does around a recording of a decode step into a graph,
shown on the host with stand-ins for the device's graph objects: nothing that a
recorded graph holds is released between the start and the end of a capture,
also when a part asks for more room in the middle of it."""
import contextlib

import pytest
import torch

from emulated_kernels import EmulatedKernels
from llm_rs_amd import Engine, LlamaConfig, StepEntry, random_model_tensors, use_kernels
from tiny_configs import TINY_A


class FakeGraph:
    capturing = False
    destroyed_while_capturing = 0
    destroyed = 0

    def replay(self):
        pass

    def __del__(self):
        FakeGraph.destroyed += 1
        if FakeGraph.capturing:
            FakeGraph.destroyed_while_capturing += 1


@contextlib.contextmanager
def fake_capture(graph):
    FakeGraph.capturing = True
    try:
        yield
    finally:
        FakeGraph.capturing = False


@pytest.fixture
def engine(monkeypatch):
    FakeGraph.capturing, FakeGraph.destroyed_while_capturing, FakeGraph.destroyed = False, 0, 0
    monkeypatch.setattr(torch.cuda, "CUDAGraph", FakeGraph)
    monkeypatch.setattr(torch.cuda, "graph", fake_capture)
    cfg = LlamaConfig.from_dict(TINY_A)
    with use_kernels(EmulatedKernels()):
        e = Engine(cfg, random_model_tensors(cfg, 3), dtype="float32", device="cpu", page_size=4, num_pages=64, max_requests=4)
        e.runner.use_graphs = True      # as on the device
        yield e


def _decode(engine, slots, pos):
    out = engine.step([StepEntry(s, pos[s], [7 + s], [0]) for s in slots])
    for s in slots:
        pos[s] += 1
    return out.clone()


def test_growth_during_a_recording_destroys_nothing_until_it_has_ended(engine):
    runner = engine.runner
    a, b = engine.open_request(), engine.open_request()
    pos = {a: 0, b: 0}
    _decode(engine, [a, b], pos)                    # eager; the buffers grow to what two rows need
    _decode(engine, [a], pos)                       # seen once: eager
    _decode(engine, [a], pos)                       # seen twice: recorded
    assert len(runner._graphs) == 1 and FakeGraph.destroyed == 0
    first_key = next(iter(runner._graphs))

    # a part that asks for more room when it is recorded than when it ran eagerly
    forward = engine.model.forward
    asked = []

    def greedy_forward(ctx, views):
        if FakeGraph.capturing:
            asked.append(ctx.n_tokens)
            ctx.workspace("toy.more", (1 << 20,), torch.float32)
            raise AssertionError("the workspace grew in the middle of a recording")
        return forward(ctx, views)

    engine.model.forward = greedy_forward
    _decode(engine, [a, b], pos)                    # seen once: eager
    eager = _decode(engine, [a, b], pos)            # recording given up, run eagerly instead
    assert asked == [2]
    assert FakeGraph.destroyed_while_capturing == 0
    assert first_key in runner._graphs and len(runner._graphs) == 1, "the graphs recorded earlier stay: no address changed"
    assert "toy.more" not in runner._buffers
    assert not runner._recording
    assert FakeGraph.destroyed == 1                 # the abandoned recording, dropped after its capture had ended
    # the step that gave its recording up still returned this step's logits
    engine.model.forward = forward
    pos_check = dict(pos)
    c = engine.open_request()
    whole = engine.step([StepEntry(c, 0, [7 + a] * pos_check[a], [pos_check[a] - 1])])
    assert torch.allclose(whole[0], eager[0], atol=1e-5)

    # outside a recording a buffer that grows does drop the graphs, which hold the old addresses
    runner.workspace("model.h", (1 << 16, 64), torch.float32)
    assert len(runner._graphs) == 0 and FakeGraph.destroyed == 2 and FakeGraph.destroyed_while_capturing == 0


def test_no_buffer_is_asked_to_grow_on_the_recording_pass(engine):
    """The eager runs of a shape make every buffer as large as its recording needs."""
    runner = engine.runner
    grown = []
    workspace = runner.workspace

    def watching(name, shape, dtype):
        before = runner._buffers.get(name)
        out = workspace(name, shape, dtype)
        if FakeGraph.capturing and runner._buffers.get(name) is not before:
            grown.append(name)
        return out

    runner.workspace = watching
    slots = [engine.open_request() for _ in range(3)]
    pos = {s: 0 for s in slots}
    for _ in range(4):
        _decode(engine, slots, pos)
    assert len(runner._graphs) == 1 and grown == []
