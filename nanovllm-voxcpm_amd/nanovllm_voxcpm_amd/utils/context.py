"""Per-domain LoRA batch context read by the LoRA linears.

Same data model and accessors as the reference's ``nanovllm_voxcpm/utils/context.py``
(``LoRAContext`` :21-34, the three domains :4-6, ``get/set/reset_lora_context`` :73-74,
127-155).  ``build_lora_context_from_token_to_slot`` (:77-116 in the reference, a Python loop
over slots with ``nonzero`` per slot) is one on-device counting sort here.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from nanovllm_voxcpm_amd import _hip
from nanovllm_voxcpm_amd.lora_ops.segment_meta import as_slot_vector

LM_LORA_DOMAIN = "lm_domain"
PROJ_LORA_DOMAIN = "proj_domain"
DIT_LORA_DOMAIN = "dit_domain"
LORA_DOMAINS = (LM_LORA_DOMAIN, PROJ_LORA_DOMAIN, DIT_LORA_DOMAIN)


@dataclass
class LoRAContext:
    token_to_slot: torch.Tensor | None = None
    token_indices_sorted_by_slot: torch.Tensor | None = None
    active_slot_ids: torch.Tensor | None = None
    num_tokens_per_slot: torch.Tensor | None = None
    slot_start_offsets: torch.Tensor | None = None
    no_lora_flag: bool = True
    num_active_loras: int = 0
    # LoRAMetadata view shared by every LoRA layer of the step (and, through it, the
    # segment plan the kernels walk); dropped whenever the context is (re)installed.
    _cached_metadata: object | None = field(default=None, repr=False, compare=False)
    # segment plans the HIP backend derived from token_to_slot (a derived array of the context,
    # like the sorted indices above): valid until the context is installed again or its buffers
    # are refreshed in place, both of which empty the table
    _segment_plans: dict = field(default_factory=dict, repr=False, compare=False)


_DOMAINS: dict[str, LoRAContext] = {}


def get_lora_context(domain: str = LM_LORA_DOMAIN) -> LoRAContext:
    ctx = _DOMAINS.get(domain)
    return ctx if ctx is not None else LoRAContext()


def set_lora_context(lora_context: LoRAContext, *, domain: str = LM_LORA_DOMAIN) -> None:
    invalidate_lora_context(lora_context)
    _DOMAINS[domain] = lora_context


def invalidate_lora_context(lora_context: LoRAContext) -> None:
    """Forget everything derived from the context's tensors (call after rewriting them in place)."""
    lora_context._cached_metadata = None
    lora_context._segment_plans.clear()


def reset_lora_context(domain: str | None = None) -> None:
    if domain is None:
        _DOMAINS.clear()
    else:
        _DOMAINS.pop(domain, None)


def build_lora_context_from_token_to_slot(
    token_to_slot: torch.Tensor | None,
    *,
    max_slots: int | None = None,
    sync: bool = True,
) -> LoRAContext:
    """Context for a slot-id vector that already lives on the GPU.

    The compact arrays leave out slot -1, list the slots in ascending order and the tokens of
    a slot in ascending order — the layout the reference's builders produce.

    ``max_slots`` bounds the slot ids (one past the largest valid id); when omitted it is read
    from the data, which costs a host synchronisation.  With ``sync=True`` two counters are
    read back so that the arrays get their exact lengths and ``no_lora_flag`` /
    ``num_active_loras`` are exact.  With ``sync=False`` nothing is read back: arrays keep
    their capacity (unused ids are -1, counts and offsets 0), ``no_lora_flag`` is False and
    ``num_active_loras`` is the bucket capacity — the form a captured graph can replay.
    """
    if token_to_slot is None or token_to_slot.numel() == 0:
        return LoRAContext(token_to_slot=token_to_slot, no_lora_flag=True, num_active_loras=0)
    if not token_to_slot.is_cuda:
        raise RuntimeError("token_to_slot must live on the GPU; the HIP LoRA path has no host fallback")
    tts = as_slot_vector(token_to_slot)
    n = tts.numel()
    if max_slots is None:
        if not sync:
            raise ValueError("max_slots is required when sync=False")
        max_slots = max(int(tts.max().item()) + 1, 1)
    cap = min(n, max_slots)
    i32 = dict(dtype=torch.int32, device=tts.device)
    sorted_idx = torch.empty(n, **i32)
    ids = torch.empty(cap, **i32)
    counts = torch.empty(cap, **i32)
    offsets = torch.empty(cap + 1, **i32)
    scalars = torch.empty(4, **i32)
    _hip.meta_build(
        tts,
        max_slots,
        sorted_idx=sorted_idx,
        compact_ids=ids,
        compact_counts=counts,
        compact_offsets=offsets,
        compact_capacity=cap,
        scalars=scalars,
    )
    if not sync:
        return LoRAContext(
            token_to_slot=tts,
            token_indices_sorted_by_slot=sorted_idx,
            active_slot_ids=ids,
            num_tokens_per_slot=counts,
            slot_start_offsets=offsets,
            no_lora_flag=False,
            num_active_loras=cap,
        )
    n_active, n_sorted, no_lora, _bad = scalars.tolist()
    if no_lora:
        return LoRAContext(token_to_slot=tts, no_lora_flag=True, num_active_loras=0)
    return LoRAContext(
        token_to_slot=tts,
        token_indices_sorted_by_slot=sorted_idx[:n_sorted],
        active_slot_ids=ids[:n_active],
        num_tokens_per_slot=counts[:n_active],
        slot_start_offsets=offsets[: n_active + 1],
        no_lora_flag=False,
        num_active_loras=n_active,
    )


def set_lora_context_from_token_to_slot(
    token_to_slot: torch.Tensor | None,
    *,
    domain: str = LM_LORA_DOMAIN,
    max_slots: int | None = None,
    sync: bool = True,
) -> None:
    set_lora_context(
        build_lora_context_from_token_to_slot(token_to_slot, max_slots=max_slots, sync=sync), domain=domain
    )
