"""Adapter lifecycle, reference counting and LRU slot residency (host bookkeeping).

The scenarios and expected values are the reference's own (tests/unit/test_lora_runtime.py:66-126,
tests/unit/test_lora_manager.py:29-175), restated against this package, plus a few invariants the
design implies (first-use admission order, tie-break of the LRU, disabled runtime)."""

from __future__ import annotations

import pytest
import torch


class _Available:
    def availability(self):
        from nanovllm_voxcpm_amd.lora import LoRAAvailability

        return LoRAAvailability(True, None)


@pytest.fixture(autouse=True)
def _backend():
    from nanovllm_voxcpm_amd.lora import set_backend_for_testing

    set_backend_for_testing(_Available())
    yield
    set_backend_for_testing(None)


def _payload(scale: float = 1.0, rank: int = 1):
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRAModelPayload, LoRAModulePayload

    module = LoRAModulePayload(lora_a=torch.eye(rank, 2), lora_b=torch.full((1, rank), scale), effective_rank=rank, scaling=scale)
    return LoRAModelPayload(modules={"linear": module}, rank=rank, alpha=scale)


def test_batch_plan_loads_slot_and_expands_tokens():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRARuntime

    rt = LoRARuntime(max_loras=2)
    a = rt.register_lora("demo", _payload())
    rt.on_sequence_enqueued(a)
    rt.on_sequence_started(a)
    loads = []
    plan = rt.build_batch_plan([a, None, a], [2, 1, 1], lambda slot, payload: loads.append((slot, payload.rank)))
    assert loads == [(0, 1)]
    assert plan.token_to_slot == [0, 0, -1, 0]
    assert plan.token_indices_sorted_by_slot == [0, 1, 3]
    assert plan.active_slot_ids == [0]
    assert plan.num_tokens_per_slot == [3]
    assert plan.slot_start_offsets == [0, 3]
    assert plan.adapter_to_slot == {a: 0}


def test_capacity_and_lru_eviction():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRARuntime

    rt = LoRARuntime(max_loras=2)
    a, b, c = (rt.register_lora(n, _payload(s)) for n, s in (("a", 1.0), ("b", 2.0), ("c", 3.0)))
    for adapter in (a, b):
        rt.on_sequence_enqueued(adapter)
        rt.on_sequence_started(adapter)
    rt.build_batch_plan([a, b], [1, 1], lambda slot, payload: None)
    assert rt.can_schedule({a, b}, c) is False
    with pytest.raises(RuntimeError, match="No idle LoRA GPU slot"):
        rt.build_batch_plan([c], [1], lambda slot, payload: None)
    rt.on_sequence_preempted(b)
    assert rt.can_schedule({a}, c) is True
    loads = []
    plan = rt.build_batch_plan([a, c], [1, 1], lambda slot, payload: loads.append((slot, payload.alpha)))
    assert loads == [(1, 3.0)]
    assert plan.active_slot_ids == [0, 1]
    assert sorted(plan.adapter_to_slot) == [a, c]
    assert rt.get_entry(b).slot_id is None and rt.get_entry(c).slot_id == 1


def test_lru_prefers_oldest_idle_slot_then_lowest_id():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRARuntime

    rt = LoRARuntime(max_loras=3)
    ids = [rt.register_lora(f"l{i}", _payload(float(i + 1))) for i in range(5)]
    loads = []
    load = lambda slot, payload: loads.append((slot, payload.alpha))  # noqa: E731
    rt.build_batch_plan(ids[:3], [1, 1, 1], load)           # slots 0,1,2 in first-use order
    rt.build_batch_plan([ids[0]], [1], load)                  # touch adapter 0: adapter 1 is now the oldest
    rt.build_batch_plan([ids[3]], [1], load)                  # evicts adapter 1 (slot 1)
    rt.build_batch_plan([ids[4]], [1], load)                  # evicts adapter 2 (slot 2)
    assert loads == [(0, 1.0), (1, 2.0), (2, 3.0), (1, 4.0), (2, 5.0)]
    assert [rt.get_entry(i).slot_id for i in ids] == [0, None, None, 1, 2]


def test_lifecycle_and_draining():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRALifecycleState, LoRAManager

    m = LoRAManager(max_loras=2)
    a = m.register_lora("demo", _payload())
    assert m.get_entry(a).state == LoRALifecycleState.REGISTERED
    m.on_sequence_enqueued(a)
    assert m.get_entry(a).state == LoRALifecycleState.ACTIVE
    m.on_sequence_started(a)
    m.on_sequence_finished(a, was_running=True)
    assert m.get_entry(a).state == LoRALifecycleState.REGISTERED
    m.unregister_lora("demo")
    assert m.list_loras() == []
    with pytest.raises(ValueError, match="not registered"):
        m.resolve_adapter("demo")


def test_manager_tracks_capacity_without_payloads():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRAManager

    m = LoRAManager(max_loras=2)
    a, b, c = (m.register_lora(n, _payload(s)) for n, s in (("a", 1.0), ("b", 2.0), ("c", 3.0)))
    for adapter in (a, b):
        m.on_sequence_enqueued(adapter)
        m.on_sequence_started(adapter)
    # nothing is resident in a manager, but two empty slots cannot take three adapters
    assert m.can_schedule({a, b}, c) is False
    m.on_sequence_preempted(b)
    assert m.can_schedule({a}, c) is True
    assert m.can_schedule({a, b}, None) is True


@pytest.mark.parametrize("running", [False, True])
def test_unregister_drains_old_requests_and_rejects_new_ones(running):
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRALifecycleState, LoRAManager

    m = LoRAManager(max_loras=1)
    a = m.register_lora("demo", _payload())
    m.on_sequence_enqueued(a)
    if running:
        m.on_sequence_started(a)
    m.unregister_lora("demo")
    entry = m.get_entry(a)
    assert entry.state == LoRALifecycleState.DRAINING
    assert entry.cpu_ref_count == 1 and entry.gpu_running_ref_count == int(running)
    with pytest.raises(ValueError, match="draining"):
        m.resolve_adapter("demo")
    m.on_sequence_finished(a, was_running=running)
    assert m.list_loras() == []


def test_fixed_adapter_ids_rank_limit_and_duplicates():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRAManager

    rank0, rank1 = LoRAManager(max_loras=1), LoRAManager(max_loras=1)
    assert rank0.register_lora("shared", _payload(1.0), adapter_id=7) == 7
    assert rank1.register_lora("shared", _payload(2.0), adapter_id=7) == 7
    assert rank0.get_entry(7).alpha == 1.0 and rank1.get_entry(7).alpha == 2.0
    assert rank0.peek_next_adapter_id() == 8
    with pytest.raises(ValueError, match="already registered"):
        rank0.register_lora("shared", _payload())
    with pytest.raises(ValueError, match="adapter id 7 is already registered"):
        rank0.register_lora("other", _payload(), adapter_id=7)
    limited = LoRAManager(max_loras=1, max_lora_rank=1)
    with pytest.raises(ValueError, match="max_lora_rank"):
        limited.register_lora("too-big", _payload(2.0, rank=2))


def test_reference_count_underflow_and_disabled_runtime():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRAManager, LoRARuntime

    m = LoRAManager(max_loras=1)
    a = m.register_lora("demo", _payload())
    with pytest.raises(RuntimeError, match="GPU ref count underflow"):
        m.on_sequence_preempted(a)
    with pytest.raises(RuntimeError, match="CPU ref count underflow"):
        m.on_sequence_finished(a, was_running=False)
    m.on_sequence_enqueued(None)  # sequences without adapter are not counted
    off = LoRARuntime(max_loras=0)
    assert off.enabled is False and off.can_schedule(set(), 3) is True
    with pytest.raises(RuntimeError, match="disabled"):
        off.register_lora("x", _payload())
    plan = off.build_batch_plan([None, None], [2, 1], lambda slot, payload: None)
    assert plan.token_to_slot == [-1, -1, -1] and plan.slot_start_offsets == [0]
    with pytest.raises(ValueError, match="same length"):
        off.build_batch_plan([None], [1, 2], lambda slot, payload: None)


def test_evicted_adapter_of_removed_entry_frees_its_slot():
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRARuntime

    rt = LoRARuntime(max_loras=1)
    a = rt.register_lora("a", _payload(1.0))
    b = rt.register_lora("b", _payload(2.0))
    rt.build_batch_plan([a], [1], lambda slot, payload: None)
    rt.unregister_lora("a")  # no requests: removed at once, slot 0 is empty again
    loads = []
    rt.build_batch_plan([b], [3], lambda slot, payload: loads.append(slot))
    assert loads == [0] and rt.get_entry(b).slot_id == 0


@pytest.mark.gpu
def test_runtime_drives_a_layer_through_eviction_on_the_gpu():
    """Requests -> runtime (admission, LRU eviction, slot loads into a real layer) -> batch plan ->
    device context -> HIP path; checked against x W^T + the adapter each sequence asked for."""
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRAModelPayload, LoRAModulePayload, LoRARuntime, build_lora_context_from_batch_plan
    from nanovllm_voxcpm_amd.layers.lora import LoRALinear
    from nanovllm_voxcpm_amd.lora import set_backend_for_testing
    from nanovllm_voxcpm_amd.utils.context import reset_lora_context, set_lora_context

    set_backend_for_testing(None)  # the real backend
    g = torch.Generator().manual_seed(5)
    k, n, rank = 64, 48, 8
    layer = LoRALinear(k, n, bias=False, max_loras=2, max_lora_rank=rank).cuda()
    with torch.no_grad():
        layer.weight.copy_(torch.randn(n, k, generator=g) * 0.1)
    adapters = {}
    rt = LoRARuntime(max_loras=2, max_lora_rank=rank)
    for name in ("a", "b", "c"):
        a, b = torch.randn(rank, k, generator=g) * 0.1, torch.randn(n, rank, generator=g) * 0.1
        payload = LoRAModelPayload({"linear": LoRAModulePayload(a, b, rank, 2.0)}, rank=rank, alpha=2.0 * rank)
        adapters[rt.register_lora(name, payload)] = (a, b)

    def load(slot, payload):
        m = payload.modules["linear"]
        layer.set_slot_lora(slot, m.lora_a.cuda(), m.lora_b.cuda(), m.effective_rank, m.scaling)

    for batch in ([0, 1, None], [0, 2, None, 2], [1, None]):  # the second batch evicts b, the third brings it back
        counts = [3 if a is not None else 2 for a in batch]
        plan = rt.build_batch_plan(batch, counts, load)
        x = torch.randn(sum(counts), k, generator=g)
        set_lora_context(build_lora_context_from_batch_plan(plan, max_slots=2))
        try:
            got = layer(x.cuda()).cpu()
        finally:
            reset_lora_context()
        want = x @ layer.weight.detach().cpu().T
        row = 0
        for adapter, count in zip(batch, counts):
            if adapter is not None:
                a, b = adapters[adapter]
                want[row : row + count] += (x[row : row + count] @ a.T) @ b.T * 2.0
            row += count
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)
