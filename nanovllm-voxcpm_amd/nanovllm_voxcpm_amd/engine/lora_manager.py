"""Batch plan -> device LoRA context, with the segment arrays built on the GPU.

Counterpart of the index builders of the reference's ``nanovllm_voxcpm/engine/lora_manager.py``
(:67-180).  The reference sorts the tokens by slot in Python for every step and domain
(:77-91) and uploads five packed arrays (:118-176); here only the slot-id vector crosses PCIe
(one pinned copy) and one launch of the on-device counting sort produces the rest.  The
adapter lifecycle / LRU residency half of that file lives in ``lora_runtime.py`` and is
re-exported here under the reference's import path.
"""

from __future__ import annotations

import torch

from nanovllm_voxcpm_amd import _hip
from nanovllm_voxcpm_amd.utils.context import LoRAContext


class LoRABatchPlan:
    """What the scheduler knows on the host: which slot every token of the batch uses.

    Takes the six fields of the reference's dataclass (lora_manager.py:67-75) in its order; the
    four segment arrays may be left out and are then derived from ``token_to_slot`` on demand
    (the device path never reads them: the GPU sorts the tokens itself)."""

    __slots__ = ("adapter_to_slot", "token_to_slot", "_sorted", "_active", "_counts", "_offsets")

    def __init__(
        self,
        adapter_to_slot: dict[int, int],
        token_to_slot: list[int],
        token_indices_sorted_by_slot: list[int] | None = None,
        active_slot_ids: list[int] | None = None,
        num_tokens_per_slot: list[int] | None = None,
        slot_start_offsets: list[int] | None = None,
    ) -> None:
        self.adapter_to_slot = adapter_to_slot
        self.token_to_slot = token_to_slot
        self._sorted = token_indices_sorted_by_slot
        self._active = active_slot_ids
        self._counts = num_tokens_per_slot
        self._offsets = slot_start_offsets

    def __repr__(self) -> str:
        return f"LoRABatchPlan(adapter_to_slot={self.adapter_to_slot!r}, token_to_slot={self.token_to_slot!r})"

    def __eq__(self, other) -> bool:
        if not isinstance(other, LoRABatchPlan):
            return NotImplemented
        return self.adapter_to_slot == other.adapter_to_slot and list(self.token_to_slot) == list(other.token_to_slot)

    @property
    def num_lora_tokens(self) -> int:
        return sum(1 for s in self.token_to_slot if s >= 0)

    @property
    def active_slot_ids(self) -> list[int]:
        if self._active is None:
            self._active = sorted({s for s in self.token_to_slot if s >= 0})
        return self._active

    @property
    def num_tokens_per_slot(self) -> list[int]:
        if self._counts is None:
            self._counts = [sum(1 for s in self.token_to_slot if s == slot) for slot in self.active_slot_ids]
        return self._counts

    @property
    def slot_start_offsets(self) -> list[int]:
        if self._offsets is None:
            offsets = [0]
            for count in self.num_tokens_per_slot:
                offsets.append(offsets[-1] + count)
            self._offsets = offsets
        return self._offsets

    @property
    def token_indices_sorted_by_slot(self) -> list[int]:
        if self._sorted is None:
            keyed = [(s, t) for t, s in enumerate(self.token_to_slot) if s >= 0]
            self._sorted = [t for _, t in sorted(keyed)]
        return self._sorted


def build_lora_batch_plan_from_token_to_slot(
    adapter_to_slot: dict[int, int],
    token_to_slot: list[int],
) -> LoRABatchPlan:
    return LoRABatchPlan(adapter_to_slot=adapter_to_slot, token_to_slot=list(token_to_slot))


def expand_token_to_slot(adapter_slots: list[int], token_counts: list[int]) -> list[int]:
    """Per-sequence slot ids repeated per token (reference: lora_manager.py:399-403)."""
    if len(adapter_slots) != len(token_counts):
        raise ValueError("adapter_ids and token_counts must have the same length")
    out: list[int] = []
    for slot, count in zip(adapter_slots, token_counts):
        out.extend([slot] * count)
    return out


def _upload_int32(values: list[int], device: torch.device | str) -> torch.Tensor:
    host = torch.tensor(values, dtype=torch.int32, device="cpu", pin_memory=True)
    return host.to(device, non_blocking=True)


def build_lora_context_from_batch_plan(
    plan: LoRABatchPlan,
    *,
    max_slots: int | None = None,
    device: torch.device | str = "cuda",
) -> LoRAContext:
    """One H2D copy of the slot ids, one metadata launch, no device->host traffic: the array
    lengths and the two host flags come from the host list the plan already holds."""
    slots = plan.token_to_slot
    tts = _upload_int32(slots, device) if slots else torch.empty(0, dtype=torch.int32, device=device)
    active = plan.active_slot_ids
    if not active:
        return LoRAContext(token_to_slot=tts, no_lora_flag=True, num_active_loras=0)
    n, n_lora, n_active = len(slots), plan.num_lora_tokens, len(active)
    if max_slots is None:
        max_slots = active[-1] + 1
    elif active[-1] >= max_slots:
        raise ValueError(f"slot id {active[-1]} is outside the {max_slots} resident slots")
    cap = min(n, max_slots)
    i32 = dict(dtype=torch.int32, device=tts.device)
    # one allocation, four views
    packed = torch.empty(n + 2 * cap + cap + 1, **i32)
    sorted_idx, ids, counts, offsets = packed.split([n, cap, cap, cap + 1])
    _hip.meta_build(
        tts,
        max_slots,
        sorted_idx=sorted_idx,
        compact_ids=ids,
        compact_counts=counts,
        compact_offsets=offsets,
        compact_capacity=cap,
    )
    return LoRAContext(
        token_to_slot=tts,
        token_indices_sorted_by_slot=sorted_idx[:n_lora],
        active_slot_ids=ids[:n_active],
        num_tokens_per_slot=counts[:n_active],
        slot_start_offsets=offsets[: n_active + 1],
        no_lora_flag=False,
        num_active_loras=n_active,
    )


def build_lora_context_from_slot_list(
    token_to_slot: list[int],
    *,
    max_slots: int | None = None,
    device: torch.device | str = "cuda",
) -> LoRAContext:
    return build_lora_context_from_batch_plan(
        build_lora_batch_plan_from_token_to_slot({}, token_to_slot), max_slots=max_slots, device=device
    )


from nanovllm_voxcpm_amd.engine.lora_runtime import (  # noqa: E402  (re-export under the reference's module path)
    LoRAControlEntry,
    LoRALifecycleState,
    LoRAManager,
    LoRAModelPayload,
    LoRAModulePayload,
    LoRAResidentState,
    LoRARuntime,
    LoRARuntimeEntry,
    LoRASlot,
)
