"""Segment metadata built on the GPU from the per-token slot-id vector.

`SegmentPlan` is the workspace the fused apply kernels walk (tokens grouped by slot, tiles
of at most 8 / 64 tokens).  `LoRAKernelMeta` keeps the reference's buffer-holding dataclass
and field names (reference: nanovllm_voxcpm/lora_ops/triton_ops/lora_kernel_metadata.py:9-79)
but fills every buffer with one launch of the on-device counting sort instead of
sort / unique / cumsum plus a host read-back per call.
"""

from __future__ import annotations

import bisect
from dataclasses import dataclass, field

import torch

from nanovllm_voxcpm_amd import _hip


def as_slot_vector(token_to_slot: torch.Tensor) -> torch.Tensor:
    """The slot ids as the contiguous int32 vector the kernels read."""
    if token_to_slot.dtype != torch.int32:
        token_to_slot = token_to_slot.to(torch.int32)
    return token_to_slot if token_to_slot.is_contiguous() else token_to_slot.contiguous()


@dataclass
class SegmentPlan:
    """Device workspace produced by one metadata launch for one slot-id vector."""

    workspace: torch.Tensor  # int32, layout documented in include/mlora.h
    token_to_slot: torch.Tensor  # the int32 vector the plan was built from (kept alive)
    num_tokens: int
    max_slots: int

    def header(self) -> list[int]:
        """Header words copied to the host (synchronises; diagnostics and tests only)."""
        return self.workspace[: _hip.PLAN_HEADER_WORDS].tolist()

    def rejected_launches(self) -> int:
        """How many launches found this plan built for another batch shape (or not built at all)
        and therefore left y untouched.  The C-ABI returns 0 for such a launch - only the device
        sees the mismatch - so a native caller that reuses plans checks this word; the Python
        boundary builds its plans itself and never gets there.  Synchronises."""
        return int(self.workspace[_hip.PLAN_REJECTED].item())


def build_segment_plan(token_to_slot: torch.Tensor, max_slots: int) -> SegmentPlan:
    """Group the tokens by slot on the device; no host synchronisation."""
    tts = as_slot_vector(token_to_slot)
    if max_slots > _hip.MAX_SLOTS:
        raise ValueError(f"max_slots={max_slots} exceeds the supported {_hip.MAX_SLOTS}")
    words = _hip.plan_workspace_words(tts.numel(), max_slots)
    workspace = torch.empty(words, dtype=torch.int32, device=tts.device)
    _hip.meta_build(tts, max_slots, plan=workspace)
    return SegmentPlan(workspace=workspace, token_to_slot=tts, num_tokens=tts.numel(), max_slots=max_slots)


@dataclass
class LoRAKernelMeta:
    """Preallocated index buffers in the layout of the reference's grouped kernels.

    Unlike the plan above, the "no LoRA" tokens (slot -1) form the first bucket of
    ``token_indices_sorted_by_lora_ids`` / ``active_lora_ids``; unused bucket entries hold
    id -1, count 0 and start 0.
    """

    token_lora_mapping: torch.Tensor
    token_indices_sorted_by_lora_ids: torch.Tensor
    active_lora_ids: torch.Tensor
    num_tokens_per_lora: torch.Tensor
    lora_token_start_loc: torch.Tensor
    no_lora_flag: bool = False
    num_active_loras: int = 0
    default_num_active_loras: int = 0
    captured_lora_counts: list[int] = field(default_factory=list)
    _scalars: torch.Tensor | None = field(default=None, repr=False)

    @staticmethod
    def make(
        max_loras: int,
        max_num_tokens: int,
        device: torch.device | str,
        captured_lora_counts: list[int] | None = None,
    ) -> "LoRAKernelMeta":
        i32 = dict(dtype=torch.int32, device=device)
        return LoRAKernelMeta(
            token_lora_mapping=torch.empty(max_num_tokens, **i32),
            token_indices_sorted_by_lora_ids=torch.empty(max_num_tokens, **i32),
            active_lora_ids=torch.full((max_loras + 1,), -1, **i32),
            num_tokens_per_lora=torch.zeros(max_loras + 1, **i32),
            lora_token_start_loc=torch.zeros(max_loras + 2, **i32),
            default_num_active_loras=max_loras + 1,
            captured_lora_counts=sorted(captured_lora_counts) if captured_lora_counts else [],
            _scalars=torch.zeros(4, **i32),
        )

    @property
    def max_loras(self) -> int:
        return self.active_lora_ids.numel() - 1

    def prepare_tensors(self, token_lora_mapping: torch.Tensor, *, sync: bool = True) -> None:
        """Fill every buffer for this batch.

        ``sync=True`` reads two integers back so that ``no_lora_flag`` and
        ``num_active_loras`` are exact, as the reference's are.  ``sync=False`` performs no
        host read (safe under graph capture) and reports the conservative values
        ``no_lora_flag=False`` and ``num_active_loras=max_loras + 1``.
        """
        tts = as_slot_vector(token_lora_mapping)
        n = tts.numel()
        if n > self.token_lora_mapping.numel():
            raise ValueError(f"{n} tokens exceed the capacity {self.token_lora_mapping.numel()} of this LoRAKernelMeta")
        self.no_lora_flag = False
        self.num_active_loras = 0
        if n == 0:
            # torch.all() of an empty mask is True in the reference: nothing to run.
            self.active_lora_ids.fill_(-1)
            self.num_tokens_per_lora.zero_()
            self.lora_token_start_loc.zero_()
            self.no_lora_flag = True
            return
        _hip.meta_build(
            tts,
            self.max_loras,
            no_lora_bucket=True,
            sorted_idx=self.token_indices_sorted_by_lora_ids,
            compact_ids=self.active_lora_ids,
            compact_counts=self.num_tokens_per_lora,
            compact_offsets=self.lora_token_start_loc,
            compact_capacity=self.max_loras + 1,
            scalars=self._scalars,
        )
        self.token_lora_mapping[:n].copy_(tts, non_blocking=True)
        if not sync:
            self.num_active_loras = self.default_num_active_loras
            return
        n_buckets, _, no_lora, _ = self._scalars.tolist()
        self.no_lora_flag = bool(no_lora)
        if self.no_lora_flag:
            return
        num_active = n_buckets
        if self.captured_lora_counts and num_active > 0:
            idx = bisect.bisect_left(self.captured_lora_counts, num_active)
            if idx < len(self.captured_lora_counts):
                num_active = self.captured_lora_counts[idx]
        self.num_active_loras = num_active

    def meta_args(self, token_nums: int, specialize_active_lora: bool):
        num_active = self.num_active_loras if specialize_active_lora else self.default_num_active_loras
        return (
            self.token_lora_mapping[:token_nums],
            self.token_indices_sorted_by_lora_ids[:token_nums],
            self.num_tokens_per_lora,
            self.lora_token_start_loc,
            self.active_lora_ids,
            self.no_lora_flag,
            num_active,
        )
