"""Adapter registry, request reference counting and LRU residency of the GPU slots.

Host bookkeeping that turns "these sequences use these adapters" into the per-token slot
vector the kernels consume.  Same public surface and behaviour as the reference's
``LoRAManager`` / ``LoRARuntime`` (nanovllm_voxcpm/engine/lora_manager.py:13-66, 183-455):

* lifecycle of a registered adapter: REGISTERED <-> ACTIVE while requests hold it (cpu refs),
  DRAINING after ``unregister_lora`` until the last request is gone, then removed;
* a slot is ACTIVE while a running sequence uses its adapter (gpu refs), IDLE otherwise; only
  IDLE or empty slots can be reclaimed, the least recently used first (ties: lowest slot id);
* ``can_schedule`` answers whether the running set plus one candidate fits the slots;
* ``LoRARuntime.build_batch_plan`` admits the batch's adapters (loading through the caller's
  ``load_lora(slot_id, payload)``) and expands per-sequence adapters to per-token slot ids.

Written around two small tables (adapters by id, slots by index) and a logical clock; nothing
here touches the GPU.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import Callable, Iterable

import torch

from nanovllm_voxcpm_amd.lora import assert_available as assert_lora_available


class LoRALifecycleState(str, Enum):
    REGISTERED = "REGISTERED"
    ACTIVE = "ACTIVE"
    DRAINING = "DRAINING"
    REMOVED = "REMOVED"


class LoRAResidentState(str, Enum):
    ACTIVE = "ACTIVE"
    IDLE = "IDLE"


@dataclass
class LoRAModulePayload:
    lora_a: torch.Tensor
    lora_b: torch.Tensor | list[torch.Tensor]
    effective_rank: int
    scaling: float


@dataclass
class LoRAModelPayload:
    modules: dict[str, LoRAModulePayload]
    rank: int
    alpha: float


@dataclass
class LoRAControlEntry:
    name: str
    adapter_id: int
    state: LoRALifecycleState
    rank: int
    alpha: float
    scaling: float
    cpu_ref_count: int = 0
    gpu_running_ref_count: int = 0
    slot_id: int | None = None
    last_used_ts: int = 0


@dataclass
class LoRARuntimeEntry(LoRAControlEntry):
    model_payload: LoRAModelPayload | None = None


@dataclass
class LoRASlot:
    slot_id: int
    adapter_id: int | None = None
    resident_state: LoRAResidentState = LoRAResidentState.IDLE
    last_used_ts: int = 0


def _residency(entry: LoRAControlEntry) -> LoRAResidentState:
    return LoRAResidentState.ACTIVE if entry.gpu_running_ref_count > 0 else LoRAResidentState.IDLE


class _LoRAStateBase:
    """Registry + reference counts + slot states; subclasses decide what an entry stores."""

    def __init__(self, max_loras: int, max_lora_rank: int | None = None):
        self.max_loras = max_loras if max_loras > 0 else 0
        self.max_lora_rank = max_lora_rank
        self._next_adapter_id = 0
        self._clock = 0
        self._name_to_adapter_id: dict[str, int] = {}
        self._entries: dict[int, LoRAControlEntry] = {}
        self._slots = [LoRASlot(slot_id=i) for i in range(self.max_loras)]

    # -- registry ---------------------------------------------------------------------------
    @property
    def enabled(self) -> bool:
        return self.max_loras > 0

    def peek_next_adapter_id(self) -> int:
        return self._next_adapter_id

    def _make_entry(self, name: str, adapter_id: int, payload: LoRAModelPayload) -> LoRAControlEntry:
        raise NotImplementedError

    def register_lora(self, name: str, payload: LoRAModelPayload, *, adapter_id: int | None = None) -> int:
        if not self.enabled:
            raise RuntimeError("LoRA runtime is disabled for this engine")
        assert_lora_available()
        if name in self._name_to_adapter_id:
            raise ValueError(f"LoRA '{name}' is already registered")
        if self.max_lora_rank is not None and payload.rank > self.max_lora_rank:
            raise ValueError(f"LoRA rank {payload.rank} exceeds max_lora_rank={self.max_lora_rank}")
        if adapter_id is None:
            adapter_id = self._next_adapter_id
        elif adapter_id in self._entries:
            raise ValueError(f"LoRA adapter id {adapter_id} is already registered")
        if adapter_id >= self._next_adapter_id:
            self._next_adapter_id = adapter_id + 1
        self._entries[adapter_id] = self._make_entry(name, adapter_id, payload)
        self._name_to_adapter_id[name] = adapter_id
        return adapter_id

    def resolve_known_adapter(self, name: str) -> int:
        adapter_id = self._name_to_adapter_id.get(name)
        if adapter_id is None:
            raise ValueError(f"LoRA '{name}' is not registered")
        return adapter_id

    def resolve_adapter(self, name: str | None) -> int | None:
        if name is None:
            return None
        adapter_id = self.resolve_known_adapter(name)
        if self._entries[adapter_id].state in (LoRALifecycleState.DRAINING, LoRALifecycleState.REMOVED):
            raise ValueError(f"LoRA '{name}' is draining and cannot accept new requests")
        return adapter_id

    def list_loras(self) -> list[LoRAControlEntry]:
        return [self._entries[i] for i in sorted(self._entries)]

    def get_entry(self, adapter_id: int) -> LoRAControlEntry:
        return self._entries[adapter_id]

    def unregister_lora(self, name: str) -> None:
        entry = self._entries[self.resolve_known_adapter(name)]
        entry.state = LoRALifecycleState.DRAINING
        if entry.cpu_ref_count == 0:
            self._drop(entry)

    def _drop(self, entry: LoRAControlEntry) -> None:
        if entry.slot_id is not None:
            self._release(self._slots[entry.slot_id])
            entry.slot_id = None
        entry.state = LoRALifecycleState.REMOVED
        self._name_to_adapter_id.pop(entry.name, None)
        self._entries.pop(entry.adapter_id, None)

    @staticmethod
    def _release(slot: LoRASlot) -> None:
        slot.adapter_id = None
        slot.resident_state = LoRAResidentState.IDLE

    # -- request reference counts ---------------------------------------------------------------
    def _counted(self, adapter_id: int | None) -> LoRAControlEntry | None:
        return None if adapter_id is None else self._entries[adapter_id]

    def _drop_gpu_ref(self, entry: LoRAControlEntry) -> None:
        if entry.gpu_running_ref_count <= 0:
            raise RuntimeError(f"LoRA adapter {entry.adapter_id} GPU ref count underflow")
        entry.gpu_running_ref_count -= 1

    def on_sequence_enqueued(self, adapter_id: int | None) -> None:
        entry = self._counted(adapter_id)
        if entry is None:
            return
        entry.cpu_ref_count += 1
        if entry.state == LoRALifecycleState.REGISTERED:
            entry.state = LoRALifecycleState.ACTIVE

    def on_sequence_started(self, adapter_id: int | None) -> None:
        entry = self._counted(adapter_id)
        if entry is None:
            return
        entry.gpu_running_ref_count += 1
        if entry.state == LoRALifecycleState.REGISTERED:
            entry.state = LoRALifecycleState.ACTIVE
        self._refresh_slot_states()

    def on_sequence_preempted(self, adapter_id: int | None) -> None:
        entry = self._counted(adapter_id)
        if entry is None:
            return
        self._drop_gpu_ref(entry)
        self._refresh_slot_states()

    def on_sequence_finished(self, adapter_id: int | None, *, was_running: bool) -> None:
        entry = self._counted(adapter_id)
        if entry is None:
            return
        if was_running:
            self._drop_gpu_ref(entry)
        if entry.cpu_ref_count <= 0:
            raise RuntimeError(f"LoRA adapter {entry.adapter_id} CPU ref count underflow")
        entry.cpu_ref_count -= 1
        self._refresh_slot_states()
        if entry.cpu_ref_count == 0:
            if entry.state == LoRALifecycleState.DRAINING:
                self._drop(entry)
            else:
                entry.state = LoRALifecycleState.REGISTERED

    # -- slots ----------------------------------------------------------------------------------
    def _refresh_slot_states(self) -> None:
        for slot in self._slots:
            if slot.adapter_id is None:
                continue
            entry = self._entries.get(slot.adapter_id)
            if entry is None:
                self._release(slot)
            else:
                slot.resident_state = _residency(entry)

    def _reclaimable(self, keep: Iterable[int]) -> list[LoRASlot]:
        """Occupied slots that may be given to another adapter: idle and not in ``keep``."""
        keep = set(keep)
        return [s for s in self._slots
                if s.adapter_id is not None and s.adapter_id not in keep and s.resident_state == LoRAResidentState.IDLE]

    def can_schedule(self, running_adapter_ids: set[int], candidate_adapter_id: int | None) -> bool:
        if not self.enabled or candidate_adapter_id is None:
            return True
        needed = set(running_adapter_ids) | {candidate_adapter_id}
        resident = {s.adapter_id for s in self._slots if s.adapter_id is not None}
        empty = sum(1 for s in self._slots if s.adapter_id is None)
        return len(needed - resident) <= empty + len(self._reclaimable(needed))

    def _tick(self) -> int:
        self._clock += 1
        return self._clock


class LoRAManager(_LoRAStateBase):
    """Control-plane view: tracks names, states and capacity without holding any weights."""

    def _make_entry(self, name: str, adapter_id: int, payload: LoRAModelPayload) -> LoRAControlEntry:
        return LoRAControlEntry(name=name, adapter_id=adapter_id, state=LoRALifecycleState.REGISTERED, rank=payload.rank,
                                alpha=payload.alpha, scaling=payload.alpha / payload.rank if payload.rank > 0 else 0.0)


class LoRARuntime(_LoRAStateBase):
    """Worker-side view: keeps the payloads and decides which adapter lives in which slot."""

    def _make_entry(self, name: str, adapter_id: int, payload: LoRAModelPayload) -> LoRARuntimeEntry:
        return LoRARuntimeEntry(name=name, adapter_id=adapter_id, state=LoRALifecycleState.REGISTERED, rank=payload.rank,
                                alpha=payload.alpha, scaling=payload.alpha / payload.rank if payload.rank > 0 else 0.0,
                                model_payload=payload)

    def get_entry(self, adapter_id: int) -> LoRARuntimeEntry:
        return self._entries[adapter_id]  # type: ignore[return-value]

    def build_batch_plan(
        self,
        adapter_ids: list[int | None],
        token_counts: list[int],
        load_lora: Callable[[int, LoRAModelPayload], None],
    ):
        """Admit the adapters of a batch and return its ``LoRABatchPlan`` (one adapter id, or
        None, and one token count per sequence)."""
        from nanovllm_voxcpm_amd.engine.lora_manager import build_lora_batch_plan_from_token_to_slot, expand_token_to_slot

        if len(adapter_ids) != len(token_counts):
            raise ValueError("adapter_ids and token_counts must have the same length")
        if not self.enabled:
            return build_lora_batch_plan_from_token_to_slot({}, [-1] * sum(token_counts))
        self._refresh_slot_states()
        adapter_to_slot: dict[int, int] = {}
        for adapter_id in dict.fromkeys(a for a in adapter_ids if a is not None):  # first-use order
            entry = self.get_entry(adapter_id)
            slot = self._slots[self._admit(entry, load_lora)]
            adapter_to_slot[adapter_id] = slot.slot_id
            entry.last_used_ts = slot.last_used_ts = self._tick()
            slot.resident_state = _residency(entry)
        per_sequence = [adapter_to_slot.get(a, -1) if a is not None else -1 for a in adapter_ids]
        return build_lora_batch_plan_from_token_to_slot(adapter_to_slot, expand_token_to_slot(per_sequence, token_counts))

    def _admit(self, entry: LoRARuntimeEntry, load_lora: Callable[[int, LoRAModelPayload], None]) -> int:
        """Slot of ``entry``, loading it into an empty slot or over the least recently used idle
        adapter when it is not resident."""
        if entry.slot_id is not None:
            return entry.slot_id
        slot = next((s for s in self._slots if s.adapter_id is None), None)
        if slot is None:
            slot = self._select_victim({entry.adapter_id})
            if slot is None:
                raise RuntimeError("No idle LoRA GPU slot available for admission")
            self._evict_slot(slot)
        if entry.model_payload is None:
            raise RuntimeError(f"LoRA runtime entry {entry.adapter_id} is missing model payload")
        load_lora(slot.slot_id, entry.model_payload)
        slot.adapter_id = entry.adapter_id
        slot.resident_state = _residency(entry)
        entry.slot_id = slot.slot_id
        entry.last_used_ts = slot.last_used_ts = self._tick()
        return slot.slot_id

    def _select_victim(self, protected_adapter_ids: set[int]) -> LoRASlot | None:
        return min(self._reclaimable(protected_adapter_ids), key=lambda s: (s.last_used_ts, s.slot_id), default=None)

    def _evict_slot(self, slot: LoRASlot) -> None:
        if slot.adapter_id is None:
            return
        entry = self.get_entry(slot.adapter_id)
        if entry.gpu_running_ref_count > 0:
            raise RuntimeError("Cannot evict ACTIVE LoRA slot")
        entry.slot_id = None
        self._release(slot)
