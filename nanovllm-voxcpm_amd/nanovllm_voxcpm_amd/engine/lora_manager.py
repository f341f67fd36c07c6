"""Batch plan -> device LoRA context, with the segment arrays built on the GPU.

Counterpart of the index builders of the reference's ``nanovllm_voxcpm/engine/lora_manager.py``
(:67-180).  The reference sorts the tokens by slot in Python for every step and domain
(:77-91) and uploads five packed arrays (:118-176); here only the slot-id vector crosses PCIe
(one pinned copy) and one launch of the on-device counting sort produces the rest.  The
adapter lifecycle / LRU residency half of that file lives in ``lora_runtime.py`` and is
re-exported here under the reference's import path.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from nanovllm_voxcpm_amd import _hip
from nanovllm_voxcpm_amd.utils.context import LoRAContext


@dataclass
class LoRABatchPlan:
    """What the scheduler knows on the host: which slot every token of the batch uses."""

    adapter_to_slot: dict[int, int]
    token_to_slot: list[int]

    @property
    def num_lora_tokens(self) -> int:
        return sum(1 for s in self.token_to_slot if s >= 0)

    @property
    def active_slot_ids(self) -> list[int]:
        return sorted({s for s in self.token_to_slot if s >= 0})

    # The remaining host-side views of the reference's plan (lora_manager.py:67-91) are derived
    # on demand; the device path never reads them (the GPU sorts the tokens itself).
    @property
    def num_tokens_per_slot(self) -> list[int]:
        return [sum(1 for s in self.token_to_slot if s == slot) for slot in self.active_slot_ids]

    @property
    def slot_start_offsets(self) -> list[int]:
        offsets = [0]
        for count in self.num_tokens_per_slot:
            offsets.append(offsets[-1] + count)
        return offsets

    @property
    def token_indices_sorted_by_slot(self) -> list[int]:
        keyed = [(s, t) for t, s in enumerate(self.token_to_slot) if s >= 0]
        return [t for _, t in sorted(keyed)]


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
