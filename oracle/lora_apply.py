"""CPU oracle for the multi-LoRA apply — TEST INFRASTRUCTURE, not product code.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module;
the shipped package never does.  Every function restates, in plain torch on the host, what
the reference computes; citations are into the reference tree.

Pinned by (tests/test_oracle_golden.py, tests/golden/*.json):
  per_token_add_lora     — closed-form outputs of the reference's own layer tests
                           (tests/unit/test_lora_layers.py:138-183, 273-308, 186-233;
                           tests/unit/test_lora_cuda.py:135-189, 576-615, 670-764, 804-833)
                           and of its backend-orchestration tests
                           (tests/unit/test_lora_runtime.py:129-259)
  fused_add_lora / fused_delta / grouped_delta — agreement with per_token_add_lora (and with
                           each other) in fp64 on random inputs, the same closed forms,
                           linearity in B and pass-through of slot -1 rows
  lora_shrink / lora_expand — the reference's own expected-value formula
                           (tests/unit/test_lora_cuda.py:868-870, 907-909) and the fake ops of
                           tests/unit/test_lora_runtime.py:136-154
No function here is "parity unpinned".
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def per_token_add_lora(
    y_slices: list[torch.Tensor],
    x: torch.Tensor,
    lora_a_slices: list[torch.Tensor],
    lora_b_slices: list[torch.Tensor],
    *,
    indices: torch.Tensor,
    scaling: float,
    y_packed: torch.Tensor | None = None,
) -> list[torch.Tensor]:
    """The reference's torch formulation of the apply, token by token, in the tensors' dtype.

    Follows _FakePunicaBackend.add_lora (reference tests/unit/test_lora_layers.py:19-48,
    identical at tests/unit/test_lora_cuda.py:24-57): for each token with slot >= 0 and each
    slice, ``hidden = F.linear(x_t, A[slot])``, ``update = F.linear(hidden, B[slot]) * scaling``,
    ``out[t] += update``.  In place iff ``y_packed`` is given, otherwise on clones.
    """
    with torch.no_grad():
        outs = list(y_slices) if y_packed is not None else [y.detach().clone() for y in y_slices]
        for t in range(x.size(0)):
            slot = int(indices[t].item())
            if slot < 0:
                continue
            for i, out in enumerate(outs):
                if out.numel() == 0:
                    continue  # empty output slices are skipped (reference nanovllm_voxcpm/lora.py:215)
                hidden = F.linear(x[t : t + 1], lora_a_slices[i][slot])
                update = F.linear(hidden, lora_b_slices[i][slot]) * scaling
                out[t : t + 1].add_(update)
    return outs


def fused_delta(
    x: torch.Tensor,
    lora_a: torch.Tensor,
    lora_b: torch.Tensor,
    indices: torch.Tensor,
    scaling: float,
    accumulate: torch.dtype = torch.float32,
) -> torch.Tensor:
    """scaling * (x . A[slot]^T) . B[slot]^T per token in ``accumulate`` precision, zero rows for
    slot < 0.  Vectorised: gather the slices, two batched matmuls.  This is the arithmetic
    the reference spells out as its own expected value
    (tests/unit/test_lora_cuda.py:868-870) extended by the expand product."""
    idx = indices.to(torch.int64)
    live = idx >= 0
    safe = idx.clamp(min=0)
    a = lora_a.to(accumulate)[safe]  # [T, r, K]
    b = lora_b.to(accumulate)[safe]  # [T, N, r]
    h = torch.bmm(a, x.to(accumulate).unsqueeze(-1)) * scaling  # [T, r, 1]
    delta = torch.bmm(b, h).squeeze(-1)  # [T, N]
    return delta * live.unsqueeze(-1).to(accumulate)


def grouped_delta(
    x: torch.Tensor,
    lora_a: torch.Tensor,
    lora_b: torch.Tensor,
    indices: torch.Tensor,
    scaling: float,
    accumulate: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Same quantity as ``fused_delta`` computed slot by slot (two dense matmuls per distinct
    slot), for batches where gathering a weight slice per token would not fit in memory.  The two
    are checked against each other in tests/test_oracle_golden.py."""
    idx = indices.to(torch.int64)
    out = torch.zeros(x.size(0), lora_b.size(1), dtype=accumulate)
    for slot in torch.unique(idx[idx >= 0]).tolist():
        rows = torch.nonzero(idx == slot).flatten()
        h = x[rows].to(accumulate) @ lora_a[slot].to(accumulate).T * scaling
        out[rows] = h @ lora_b[slot].to(accumulate).T
    return out


def fused_add_lora(
    y_slices: list[torch.Tensor],
    x: torch.Tensor,
    lora_a_slices: list[torch.Tensor],
    lora_b_slices: list[torch.Tensor],
    *,
    indices: torch.Tensor,
    scaling: float,
    accumulate: torch.dtype = torch.float32,
) -> list[torch.Tensor]:
    """What the fused kernel promises: fp32 (or wider) accumulation of the whole update and one
    rounding of ``y + delta`` to y's dtype; rows with slot < 0 are returned bit-identical.
    Returns new tensors."""
    outs = []
    live = (indices.to(torch.int64) >= 0).unsqueeze(-1)
    for y, a, b in zip(y_slices, lora_a_slices, lora_b_slices):
        if y.numel() == 0:
            outs.append(y.clone())
            continue
        big = x.size(0) * a.size(-2) * a.size(-1) > (1 << 26)
        delta = (grouped_delta if big else fused_delta)(x, a, b, indices, scaling, accumulate)
        updated = (y.to(accumulate) + delta).to(y.dtype)
        outs.append(torch.where(live, updated, y))
    return outs


def lora_shrink(
    inputs: torch.Tensor,
    lora_a_weights: list[torch.Tensor],
    token_lora_mapping: torch.Tensor,
    scaling: float,
    out_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """[S, T, r] = scaling * inputs . A_i[slot]^T, fp32 accumulate, rounded to the output
    buffer's dtype; rows with slot < 0 are zero because the reference zero-fills the buffer
    (nanovllm_voxcpm/lora_ops/triton_ops/lora_shrink_op.py:295) and its kernel applies the
    scaling before the store (kernel_utils.py:136)."""
    out_dtype = out_dtype or inputs.dtype
    outs = []
    idx = token_lora_mapping.to(torch.int64)
    live = (idx >= 0).unsqueeze(-1)
    for a in lora_a_weights:
        a3 = a.squeeze(1) if a.ndim == 4 else a
        rows = a3.to(torch.float32)[idx.clamp(min=0)]  # [T, r, K]
        h = torch.bmm(rows, inputs.to(torch.float32).unsqueeze(-1)).squeeze(-1) * scaling
        outs.append((h * live).to(out_dtype))
    return torch.stack(outs)


def lora_expand(
    inputs: torch.Tensor,
    lora_b_weights: list[torch.Tensor],
    output_tensor: torch.Tensor,
    token_lora_mapping: torch.Tensor,
    offset_start: int = 0,
    add_inputs: bool = False,
) -> torch.Tensor:
    """Returns the updated copy of ``output_tensor``: for rows with slot >= 0, column block i
    (+)= round_to_B_dtype(inputs[i] . B_i[slot]^T); the intermediate is first cast to B's dtype
    (CAST_TYPE) and the sum is formed in that dtype
    (nanovllm_voxcpm/lora_ops/triton_ops/kernel_utils.py:219-228, lora_expand_op.py:125)."""
    out = output_tensor.clone()
    idx = token_lora_mapping.to(torch.int64)
    live = (idx >= 0).unsqueeze(-1)
    col = offset_start
    for i, b in enumerate(lora_b_weights):
        b3 = b.squeeze(1) if b.ndim == 4 else b
        n = b3.size(1)
        rows = b3.to(torch.float32)[idx.clamp(min=0)]  # [T, n, r]
        h = inputs[i].to(b3.dtype).to(torch.float32)
        prod = torch.bmm(rows, h.unsqueeze(-1)).squeeze(-1).to(b3.dtype)
        block = out[:, col : col + n]
        new = (block.to(torch.float32) + prod.to(torch.float32)).to(out.dtype) if add_inputs else prod.to(out.dtype)
        out[:, col : col + n] = torch.where(live, new, block)
        col += n
    return out


class OracleBackend:
    """``LoRABackend`` stand-in that runs the reference's per-token torch loop on the host.

    Installed only by tests (through ``set_backend_for_testing``) to exercise the host logic of
    the LoRA layers without a GPU, exactly as the reference's CPU tests install their fake
    backend (reference tests/unit/test_lora_layers.py:51-57)."""

    def availability(self):
        from nanovllm_voxcpm_amd.lora import LoRAAvailability

        return LoRAAvailability(available=True, reason=None)

    def shrink(self, x, lora_a):
        return F.linear(x, lora_a)

    def expand(self, hidden, lora_b, *, scaling):
        return F.linear(hidden, lora_b) * scaling

    def add_lora(self, y_slices, x, lora_a_slices, lora_b_slices, *, indices, metadata, scaling, y_packed=None):
        return per_token_add_lora(
            y_slices, x, lora_a_slices, lora_b_slices, indices=indices, scaling=scaling, y_packed=y_packed
        )
