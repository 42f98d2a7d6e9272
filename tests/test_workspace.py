"""The arena layout of a step's buffers (no GPU): the reference's own vectors, what is
refused, and the record-then-plan behaviour of the step workspace on CPU tensors."""
import pytest
import torch

from edge_infer_amd.cache.workspace import ArenaLayout, Lifetime, Placement, lay_out
from edge_infer_amd.parts.base import Workspace


def build(*requests):
    return lay_out(Lifetime(*request) for request in requests)


def test_reference_vectors():
    """operators/tests/decode_workspace_plan_test.cpp:16-60."""
    plan = build(("residual", 1024, 0, 2), ("attn_proj", 1024, 3, 4))
    assert plan.arena_bytes == 1024 and plan.offset("residual") == plan.offset("attn_proj")
    plan = build(("q_buf", 1024, 0, 3), ("k_buf", 1024, 2, 4))
    assert plan.arena_bytes == 2048 and plan.offset("q_buf") != plan.offset("k_buf")
    plan = build(("small", 300, 0, 0, 256), ("aligned", 512, 1, 1, 512))
    assert plan.offset("small") % 256 == 0 and plan.offset("aligned") % 512 == 0
    plan = build(("large_1", 1024, 0, 0), ("small_mid", 256, 1, 1), ("large_2", 1024, 2, 2))
    assert plan.arena_bytes == 1024
    assert plan.offset("large_1") == plan.offset("small_mid") == plan.offset("large_2")


def test_a_last_use_at_the_new_first_use_still_overlaps():
    plan = build(("a", 512, 0, 2), ("b", 512, 2, 3))
    assert plan.offset("a") != plan.offset("b")
    plan = build(("a", 512, 0, 1), ("b", 512, 2, 3))
    assert plan.offset("a") == plan.offset("b")


def test_smallest_dead_slot_that_fits_and_metrics():
    plan = build(("big", 4096, 0, 0), ("small", 512, 0, 0), ("later", 400, 1, 1),
                 ("wide", 3000, 1, 1))
    assert plan.offset("later") == plan.offset("small")     # not the 4096 one
    assert plan.offset("wide") == plan.offset("big")
    assert plan.regions() == 2
    assert plan.bytes_asked() == 4096 + 512 + 400 + 3000
    assert plan.bytes_without_sharing() >= plan.bytes_asked()
    assert plan.bytes_saved() == plan.bytes_without_sharing() - plan.arena_bytes > 0


def test_requests_and_layouts_that_are_refused():
    for bad in (("", 8, 0, 0), ("x", 0, 0, 0), ("x", 8, 2, 1), ("x", 8, 0, 0, 3), ("x", 8, 0, 0, 0)):
        with pytest.raises(ValueError):
            build(bad)
    with pytest.raises(ValueError, match="twice"):
        build(("x", 8, 0, 0), ("x", 8, 1, 1))
    with pytest.raises(ValueError, match="live together"):
        ArenaLayout([Placement(Lifetime("a", 512, 0, 2), 0),
                     Placement(Lifetime("b", 512, 1, 3), 256)], 1024)
    with pytest.raises(ValueError, match="misaligned"):
        ArenaLayout([Placement(Lifetime("a", 512, 0, 2), 128)], 1024)
    with pytest.raises(ValueError, match="outside"):
        ArenaLayout([Placement(Lifetime("a", 512, 0, 2), 768)], 1024)
    with pytest.raises(KeyError):
        build(("a", 8, 0, 0)).offset("b")


def run_step(ws, signature, sizes=(1000, 600, 1000, 300)):
    """A step that takes a, b (releases a), c (releases b), a again, d; returns them."""
    ws.start(signature)
    a = ws.get("a", (sizes[0],), torch.float32)
    b = ws.get("b", (sizes[1],), torch.float32)
    ws.release(a)
    c = ws.get("c", (sizes[2],), torch.float32)
    ws.release("b")
    a2 = ws.get("a", (sizes[0],), torch.float32)
    d = ws.get("d", (sizes[3],), torch.bfloat16)
    ws.finish()
    return a, b, c, a2, d


def spans(*tensors):
    return [(t.data_ptr(), t.data_ptr() + t.numel() * t.element_size()) for t in tensors]


def test_the_step_workspace_records_then_shares_storage():
    ws = Workspace("cpu")
    first = run_step(ws, "s")
    unplanned = sum(t.numel() * t.element_size() for t in first[:3]) + first[4].numel() * 2
    a, b, c, a2, d = run_step(ws, "s")
    # c took a's storage (a was dead), the second a took b's or a new slot: all from one arena
    assert c.data_ptr() == a.data_ptr()
    assert ws.bytes() < unplanned
    # values live together never overlap: (a, b), (b, c), (c, a2, d)
    for group in ((a, b), (b, c), (c, a2, d)):
        ranges = sorted(spans(*group))
        assert all(x[1] <= y[0] for x, y in zip(ranges, ranges[1:]))
    # the same pointers again on the next step of that signature (what a captured graph needs)
    again = run_step(ws, "s")
    assert [t.data_ptr() for t in again] == [t.data_ptr() for t in (a, b, c, a2, d)]
    # another signature has a plan of its own in the same arena
    other = run_step(ws, "t", sizes=(10, 2000, 10, 5))
    other = run_step(ws, "t", sizes=(10, 2000, 10, 5))
    assert other[1].numel() == 2000
    back = run_step(ws, "s")
    assert [t.shape for t in back] == [t.shape for t in (a, b, c, a2, d)]


def test_a_step_that_leaves_its_recording_falls_back_to_named_buffers():
    ws = Workspace("cpu")
    run_step(ws, "s")
    ws.start("s")
    a = ws.get("a", (1000,), torch.float32)
    x = ws.get("unexpected", (50,), torch.float32)      # not what was recorded
    b = ws.get("b", (600,), torch.float32)
    a.fill_(1.0), x.fill_(2.0), b.fill_(3.0)
    assert a.sum() == 1000 and x.sum() == 100 and b.sum() == 1800   # nothing shared
    ws.finish()
    # the signature is recorded anew by the next step and planned again after it
    run_step(ws, "s")
    a, b, c, a2, d = run_step(ws, "s")
    assert c.data_ptr() == a.data_ptr()
    # a larger request than recorded is refused by the plan as well
    ws.start("s")
    big = ws.get("a", (5000,), torch.float32)
    assert big.numel() == 5000
    ws.abort()


def test_without_a_step_the_workspace_hands_out_one_buffer_per_name():
    ws = Workspace("cpu")
    a = ws.get("a", (8, 4), torch.float32)
    ws.release(a)                                        # ignored outside a step
    b = ws.get("a", (4, 4), torch.float32)
    assert a.data_ptr() == b.data_ptr()
    assert ws.get("c", (3,), torch.float32).data_ptr() != a.data_ptr()


def test_old_plans_are_dropped_and_planned_again_when_needed():
    ws = Workspace("cpu")
    for n in range(Workspace.MAX_PLANS + 3):
        run_step(ws, ("shape", n))
    assert len(ws._plans) == Workspace.MAX_PLANS and ("shape", 0) not in ws._plans
    run_step(ws, ("shape", 0))                 # recorded anew ...
    a, b, c, a2, d = run_step(ws, ("shape", 0))
    assert c.data_ptr() == a.data_ptr()        # ... and planned again
    # a step that fails in the middle leaves nothing behind
    ws.start("broken")
    ws.get("a", (10,), torch.float32)
    ws.abort()
    assert "broken" not in ws._plans
    run_step(ws, "broken")
    assert "broken" in ws._plans
