"""Fixed-address LoRA metadata buffers for captured decode graphs.

Counterpart of ``_make_graph_domain_buffers`` / ``_copy_lora_domain_to_graph_vars`` /
``_set_graph_lora_contexts`` of the reference's runner
(nanovllm_voxcpm/engine/model_runner.py:718-817).  The buffer set and its dense-by-slot layout
are the reference's; the refresh before every replay is one launch of the on-device counting
sort reading the batch's slot ids, instead of copy + fill + zero + scatter + cumsum per
domain.

Layout (``max_lora_buckets`` = resident slots + 1, bucket 0 stands for slot -1):
  token_to_slot                [max_rows]   batch slot ids, tail -1
  token_indices_sorted_by_slot [max_rows]   LoRA tokens grouped by slot; entries past the
                                            number of LoRA tokens keep their previous value
  active_slot_ids              [buckets]    -1, 0, 1, ... (fixed)
  num_tokens_per_slot          [buckets]    index slot + 1; entry 0 stays 0
  slot_start_offsets           [buckets+1]  0 followed by the running totals
"""

from __future__ import annotations

import torch

from nanovllm_voxcpm_amd import _hip
from nanovllm_voxcpm_amd.lora_ops.segment_meta import as_slot_vector
from nanovllm_voxcpm_amd.utils.context import LORA_DOMAINS, LoRAContext, get_lora_context, invalidate_lora_context, set_lora_context


def make_graph_domain_buffers(
    max_rows: int, max_lora_buckets: int, device: torch.device | str | None = None
) -> dict[str, torch.Tensor]:
    i32 = dict(dtype=torch.int32, device=device)
    return {
        "token_to_slot": torch.full((max_rows,), -1, **i32),
        "token_indices_sorted_by_slot": torch.arange(max_rows, **i32),
        "active_slot_ids": torch.arange(-1, max_lora_buckets - 1, **i32),
        "num_tokens_per_slot": torch.zeros(max_lora_buckets, **i32),
        "slot_start_offsets": torch.zeros(max_lora_buckets + 1, **i32),
    }


def copy_lora_domain_to_graph_vars(domain_vars: dict[str, torch.Tensor], context: LoRAContext) -> None:
    """Refresh one domain's buffers in place for the batch described by ``context``."""
    tts_buf = domain_vars["token_to_slot"]
    if not tts_buf.is_cuda:
        raise RuntimeError("graph LoRA buffers must live on the GPU; the HIP LoRA path has no host fallback")
    buckets = domain_vars["num_tokens_per_slot"].numel()
    if context.no_lora_flag or context.token_to_slot is None:
        source = torch.empty(0, dtype=torch.int32, device=tts_buf.device)
    else:
        source = as_slot_vector(context.token_to_slot)
        if source.numel() > tts_buf.numel():
            raise ValueError(f"{source.numel()} rows exceed the {tts_buf.numel()} rows captured for this graph")
    _hip.meta_build(
        source,
        buckets - 1,
        sorted_idx=domain_vars["token_indices_sorted_by_slot"],
        dense_counts=domain_vars["num_tokens_per_slot"],
        dense_offsets=domain_vars["slot_start_offsets"],
        padded_token_to_slot=tts_buf,
    )
    # Installed contexts that view these buffers were just rewritten in place (by a kernel, which
    # no tensor version counter sees): what they derived from the old contents is dropped.
    for domain in LORA_DOMAINS:
        installed = get_lora_context(domain)
        view = installed.token_to_slot
        if view is not None and view.is_cuda and view.numel() and view.data_ptr() == tts_buf.data_ptr():
            invalidate_lora_context(installed)


def set_graph_lora_contexts(graph_vars: dict, contexts: dict[str, LoRAContext]) -> None:
    """Refresh every domain and install contexts that view the fixed buffers."""
    for domain in LORA_DOMAINS:
        context = contexts[domain]
        domain_vars = graph_vars["lora_domains"][domain]
        copy_lora_domain_to_graph_vars(domain_vars, context)
        rows = 0 if context.token_to_slot is None else context.token_to_slot.size(0)
        set_lora_context(
            LoRAContext(
                token_to_slot=domain_vars["token_to_slot"][:rows],
                token_indices_sorted_by_slot=domain_vars["token_indices_sorted_by_slot"][:rows],
                active_slot_ids=domain_vars["active_slot_ids"],
                num_tokens_per_slot=domain_vars["num_tokens_per_slot"],
                slot_start_offsets=domain_vars["slot_start_offsets"],
                no_lora_flag=context.no_lora_flag,
                num_active_loras=domain_vars["active_slot_ids"].size(0),
            ),
            domain=domain,
        )
