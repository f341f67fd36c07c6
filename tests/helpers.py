"""Shared builders for the golden-vector tests (layer construction from a fixture case)."""

from __future__ import annotations

import json
from pathlib import Path

import torch

GOLDEN = Path(__file__).resolve().parent / "golden"
DTYPES = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def load_golden(name: str) -> dict:
    return json.loads((GOLDEN / name).read_text())


def make_layer(case: dict, device: str):
    """Instantiate the layer of a fixture case, load its base weight and install its slots."""
    import nanovllm_voxcpm_amd.layers.lora as L

    dtype = DTYPES[case["dtype"]]
    spec = dict(case["layer"])
    cls = getattr(L, spec.pop("type"))
    tp = case.get("tp")
    saved = (L._get_world_size, L._get_rank)
    if tp:
        L._get_world_size = lambda: tp["world_size"]
        L._get_rank = lambda: tp["rank"]
    try:
        layer = cls(**spec)
    finally:
        L._get_world_size, L._get_rank = saved
    layer = layer.to(device=device, dtype=dtype)
    with torch.no_grad():
        if "base_shards" in case:
            for shard, rows in case["base_shards"].items():
                layer._base_weight_loader(layer.weight, torch.tensor(rows, dtype=dtype, device=device), shard)
        elif case.get("base_weight") == "ones":
            layer.weight.fill_(1.0)
        else:
            layer.weight.zero_()
        for s in case["slots"]:
            a = torch.tensor(s["lora_a"], dtype=dtype, device=device)
            b = s["lora_b"]
            if isinstance(case["layer"].get("lora_targets", None), list) or case["layer"]["type"] in (
                "LoRAQKVParallelLinear",
                "LoRAMergedColumnParallelLinear",
            ):
                b = [torch.tensor(t, dtype=dtype, device=device) for t in b]
            else:
                b = torch.tensor(b, dtype=dtype, device=device)
            layer.set_slot_lora(slot_id=s["slot"], lora_a=a, lora_b=b, effective_rank=s["effective_rank"], scaling=s["scaling"])
        for slot in case.get("clear_slots", []):
            layer.clear_slot_lora(slot)
    return layer


def context_from_slots(token_to_slot: list[int], device: str, fields: str = "full"):
    """A LoRAContext as the reference's tests hand-build it (host arithmetic on tiny lists)."""
    from nanovllm_voxcpm_amd.utils.context import LoRAContext
    from oracle.segment_meta import engine_layout

    t = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    sorted_idx, active, counts, offsets = engine_layout(token_to_slot)
    if fields == "token_to_slot_and_active_only":
        return LoRAContext(token_to_slot=t(token_to_slot), active_slot_ids=t(active), no_lora_flag=False)
    return LoRAContext(
        token_to_slot=t(token_to_slot),
        token_indices_sorted_by_slot=t(sorted_idx),
        active_slot_ids=t(active),
        num_tokens_per_slot=t(counts),
        slot_start_offsets=t(offsets),
        no_lora_flag=not active,
        num_active_loras=len(active),
    )


def run_layer_case(case: dict, device: str):
    """Forward the case's batch through its layer under its context; returns (layer, y)."""
    from nanovllm_voxcpm_amd.utils.context import reset_lora_context, set_lora_context

    dtype = DTYPES[case["dtype"]]
    layer = make_layer(case, device)
    reset_lora_context()
    for domain, slots in case.get("other_domain_token_to_slot", {}).items():
        set_lora_context(context_from_slots(slots, device), domain=domain)
    if case["token_to_slot"] is not None:
        ctx = context_from_slots(case["token_to_slot"], device, case.get("context_fields", "full"))
        set_lora_context(ctx, domain=case["layer"].get("lora_domain", "lm_domain"))
    x = torch.tensor(case["x"], dtype=dtype, device=device)
    with torch.no_grad():
        y = layer(x)
    return layer, x, y
