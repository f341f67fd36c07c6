"""Low-level LoRA ops with the reference's call signatures
(reference: nanovllm_voxcpm/lora_ops/__init__.py:1-5), executed by the HIP library.

Both ops only read ``token_lora_mapping`` from the metadata tuple: a token's slot id is all
the per-token kernels need, so the three segment layouts the reference accepts (compact,
compact with a "no LoRA" bucket, dense graph buffers) are interchangeable here.
"""

from __future__ import annotations

import torch

from nanovllm_voxcpm_amd import _hip
from nanovllm_voxcpm_amd.lora_ops.segment_meta import (
    LoRAKernelMeta,
    SegmentPlan,
    as_slot_vector,
    build_segment_plan,
)

__all__ = ["LoRAKernelMeta", "SegmentPlan", "build_segment_plan", "lora_expand", "lora_shrink"]


def _as_3d(weight: torch.Tensor, what: str) -> torch.Tensor:
    """[slots, 1, d0, d1] -> [slots, d0, d1]; anything but a contiguous 3-D result is an error."""
    if weight.ndim == 4:
        if weight.size(1) != 1:
            raise ValueError(f"4-D {what} must have a singleton second dimension")
        weight = weight.squeeze(1)
    if weight.ndim != 3:
        raise ValueError(f"{what} must be [slots, rows, cols], got shape {tuple(weight.shape)}")
    if not weight.is_contiguous():
        raise ValueError(f"{what} must be contiguous")
    return weight


@torch.inference_mode()
def lora_shrink(
    inputs: torch.Tensor,
    lora_a_weights: list[torch.Tensor],
    output_tensor: torch.Tensor,
    token_lora_mapping: torch.Tensor,
    token_indices_sorted_by_lora_ids: torch.Tensor | None,
    num_tokens_per_lora: torch.Tensor | None,
    lora_token_start_loc: torch.Tensor | None,
    lora_ids: torch.Tensor | None,
    no_lora_flag: bool,
    num_active_loras: int,
    scaling: float,
) -> None:
    """output_tensor[i, t] = scaling * inputs[t] . A_i[slot_t]^T; rows without a slot become 0.

    Same arguments as the reference op
    (nanovllm_voxcpm/lora_ops/triton_ops/lora_shrink_op.py:257-341); returns without touching
    ``output_tensor`` when ``no_lora_flag`` is set, as the reference does.
    """
    if no_lora_flag:
        return
    weights = [_as_3d(w, "lora_a weight") for w in lora_a_weights]
    shapes = {tuple(w.shape) for w in weights}
    if len(shapes) != 1:
        raise ValueError("All LoRA A weights must have the same shape")
    x = inputs if inputs.stride(-1) == 1 else inputs.contiguous()
    if not output_tensor.is_contiguous() or output_tensor.ndim != 3:
        raise ValueError("output_tensor must be a contiguous [num_slices, num_tokens, rank] tensor")
    if output_tensor.size(0) != len(weights) or output_tensor.size(1) != x.size(0) or output_tensor.size(2) != weights[0].size(1):
        raise ValueError("output_tensor shape does not match [num_slices, num_tokens, rank]")
    _hip.shrink(x, weights, output_tensor, as_slot_vector(token_lora_mapping), float(scaling))


@torch.inference_mode()
def lora_expand(
    inputs: torch.Tensor,
    lora_b_weights: list[torch.Tensor],
    output_tensor: torch.Tensor,
    token_lora_mapping: torch.Tensor,
    token_indices_sorted_by_lora_ids: torch.Tensor | None,
    num_tokens_per_lora: torch.Tensor | None,
    lora_token_start_loc: torch.Tensor | None,
    lora_ids: torch.Tensor | None,
    no_lora_flag: bool,
    num_active_loras: int,
    offset_start: int = 0,
    add_inputs: bool = False,
) -> None:
    """output_tensor[t, cols of slice i] (+)= inputs[i, t] . B_i[slot_t]^T for rows with a slot.

    Same arguments as the reference op
    (nanovllm_voxcpm/lora_ops/triton_ops/lora_expand_op.py:94-170).
    """
    if no_lora_flag:
        return
    weights = [_as_3d(w, "lora_b weight") for w in lora_b_weights]
    if inputs.ndim != 3 or inputs.size(0) != len(weights):
        raise ValueError("inputs must be [num_slices, num_tokens, rank]")
    h = inputs if inputs.is_contiguous() else inputs.contiguous()
    if output_tensor.ndim != 2 or output_tensor.stride(1) != 1:
        raise ValueError("output_tensor must be 2-D with unit column stride")
    width = offset_start + sum(w.size(1) for w in weights)
    if width > output_tensor.size(1):
        raise ValueError(f"slices end at column {width} but output_tensor has {output_tensor.size(1)} columns")
    _hip.expand(h, weights, output_tensor, as_slot_vector(token_lora_mapping), int(offset_start), bool(add_inputs))
