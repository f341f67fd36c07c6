"""LoRA-wrapped linears: the callers of the batched apply.

Same constructors, parameter names, buffer layout and ``forward`` / ``set_slot_lora`` /
``clear_slot_lora`` / ``validate_slot_lora_payload`` surface as the reference's four modules
(nanovllm_voxcpm/layers/lora.py: QKV :244-465, merged-column :468-667, row-parallel :670-797,
plain :800-904), so model code and adapter loaders address them unchanged.  All four are one
implementation here: a layer is a base ``F.linear`` whose output columns are cut into blocks,
plus a list of LoRA targets, each adding ``(x . A_t[slot]^T) . B_t[slot]^T`` to one block.

Weight buffers: ``A = [slots, r, in]`` and ``B = [slots, out, r]`` with the adapter's
``alpha / r`` folded into B when a slot is installed; rows / columns at or above an adapter's
own rank stay zero, which is what makes rank padding numerically inert
(reference :395-417).
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.distributed as dist
import torch.nn as nn
import torch.nn.functional as F

from nanovllm_voxcpm_amd import _hip
from nanovllm_voxcpm_amd.lora import LoRAMetadata, get_backend
from nanovllm_voxcpm_amd.utils.context import LM_LORA_DOMAIN, get_lora_context

ShardId = str | int


def _get_world_size() -> int:
    return dist.get_world_size() if dist.is_available() and dist.is_initialized() else 1


def _get_rank() -> int:
    return dist.get_rank() if dist.is_available() and dist.is_initialized() else 0


def divide(numerator: int, denominator: int) -> int:
    if numerator % denominator:
        raise AssertionError(f"{numerator} is not divisible by {denominator}")
    return numerator // denominator


def set_weight_loader(param: nn.Parameter, loader) -> None:
    param.weight_loader = loader


_stream_is_capturing = getattr(torch._C, "_cuda_isCurrentStreamCapturing", None)


def _is_cuda_graph_capture() -> bool:
    # (asked on every forward: without an initialised GPU runtime nothing can be capturing, and
    # torch's own binding answers in a fraction of what the wrappers around it take)
    if not torch.cuda.is_initialized():
        return False
    return _stream_is_capturing() if _stream_is_capturing is not None else torch.cuda.is_current_stream_capturing()


class _LoRALayerBase(nn.Module):
    """Slot bookkeeping, context gating and the shared forward of all LoRA linears."""

    lora_scaling: torch.Tensor
    lora_base_scaling: torch.Tensor
    effective_lora_rank: torch.Tensor

    def __init__(self, max_loras: int, max_lora_rank: int, supports_lora: bool, lora_domain: str = LM_LORA_DOMAIN):
        super().__init__()
        self.max_loras = max_loras
        self.max_lora_rank = max_lora_rank
        self.supports_lora = supports_lora
        self.lora_domain = lora_domain
        self.register_buffer("lora_scaling", torch.zeros(max_loras), persistent=False)
        self.register_buffer("lora_base_scaling", torch.zeros(max_loras), persistent=False)
        self.register_buffer("effective_lora_rank", torch.zeros(max_loras, dtype=torch.int32), persistent=False)
        # host mirrors: the forward gate must never read the device
        self._lora_scaling_values = [0.0] * max_loras
        self._lora_base_scaling_values = [0.0] * max_loras
        self._effective_lora_rank_values = [0] * max_loras
        self._rank_summary_of: list | None = None  # the mirror the summary below was made from
        self._rank_summary = (False, False)

    # ---- subclass contract ------------------------------------------------------------------
    def _target_keys(self) -> list:
        """Target ids in storage order; empty for single-target layers."""
        return []

    def _a_of(self, position: int) -> torch.Tensor:
        """A buffer [slots, r, in] of the target at `position`."""
        raise NotImplementedError

    def _b_of(self, position: int) -> nn.Parameter:
        raise NotImplementedError

    def _num_targets(self) -> int:
        return max(len(self._target_keys()), 1)

    # ---- gating ---------------------------------------------------------------------------
    @property
    def lora_enabled(self) -> bool:
        return self.supports_lora

    def _active_rank(self, slot_id: int) -> int:
        return self._effective_lora_rank_values[slot_id]

    def _slot_scaling(self, slot_id: int) -> float:
        return self._lora_scaling_values[slot_id]

    def _residency(self) -> tuple[bool, bool]:
        """(some slot holds an adapter, some resident adapter is below the padded rank), from the
        host mirror; walked again only when the mirror has changed (a list comparison otherwise:
        this runs on every forward)."""
        values = self._effective_lora_rank_values
        if self._rank_summary_of != values:
            resident = [rank for rank in values if rank > 0]
            self._rank_summary = (bool(resident), any(rank < self.max_lora_rank for rank in resident))
            self._rank_summary_of = list(values)
        return self._rank_summary

    def _batch_has_no_effective_rank(self, context) -> bool:
        """True iff no slot this batch can reference holds an adapter in this module.  Decided
        from the host mirrors only; a device-resident ``active_slot_ids`` is not read."""
        active = getattr(context, "active_slot_ids", None)
        if active is None or active.is_cuda:
            return not self._residency()[0]
        return not any(s >= 0 and self._effective_lora_rank_values[int(s)] > 0 for s in active.tolist())

    def _resolve_token_slots(self, x_flat: torch.Tensor) -> torch.Tensor | None:
        """The batch's slot vector, or None when this forward needs no LoRA work."""
        if not self.supports_lora:
            return None
        context = get_lora_context(self.lora_domain)
        token_to_slot = context.token_to_slot
        if token_to_slot is None or context.no_lora_flag or token_to_slot.numel() == 0:
            return None
        if token_to_slot.device != x_flat.device:
            raise RuntimeError("LoRA token_to_slot must be prepared on the execution device by the model runner")
        if token_to_slot.numel() != x_flat.size(0):
            raise RuntimeError(
                "LoRA token_to_slot length does not match flattened input rows: "
                f"token_to_slot={token_to_slot.numel()} rows={x_flat.size(0)}"
            )
        # Never skip while a graph is being captured: the captured launches must exist for
        # adapters installed after capture.
        if not _is_cuda_graph_capture() and self._batch_has_no_effective_rank(context):
            return None
        return token_to_slot

    def _runtime_metadata(self) -> LoRAMetadata | None:
        context = get_lora_context(self.lora_domain)
        if context.token_to_slot is None:
            return None
        meta = context._cached_metadata
        # (a field assigned on the installed context without installing it again, as the
        # reference's mutable dataclass allows, makes the cached view stale: compared by identity)
        if meta is not None and (meta.token_to_slot is not context.token_to_slot or meta.no_lora_flag != context.no_lora_flag):
            context._segment_plans.clear()
            meta = None
        if meta is None:
            meta = LoRAMetadata(
                token_to_slot=context.token_to_slot,
                token_indices_sorted_by_slot=context.token_indices_sorted_by_slot,
                active_slot_ids=context.active_slot_ids,
                num_tokens_per_slot=context.num_tokens_per_slot,
                slot_start_offsets=context.slot_start_offsets,
                no_lora_flag=context.no_lora_flag,
                num_active_loras=context.num_active_loras,
            )
            # the context's own table of segment plans travels with the view (frozen dataclass)
            object.__setattr__(meta, "_mlora_context_plans", context._segment_plans)
            context._cached_metadata = meta
        return meta  # type: ignore[return-value]

    # ---- the LoRA half of forward -------------------------------------------------------------
    def _add_lora(self, x: torch.Tensor, base_out: torch.Tensor, block_sizes: list[int], block_of_target: list[int]):
        """Add every target's update to its column block of ``base_out``.

        ``block_sizes`` are the widths of the output column blocks, ``block_of_target[p]`` is
        the block the target at storage position ``p`` writes.
        """
        x_flat = x if x.ndim == 2 else x.reshape(-1, x.size(-1))
        token_to_slot = self._resolve_token_slots(x_flat)
        if token_to_slot is None:
            return base_out
        out_flat = base_out if base_out.ndim == 2 else base_out.reshape(-1, base_out.size(-1))
        a_slices = [self._a_of(p) for p in range(len(block_of_target))]
        b_slices = [self._b_of(p) for p in range(len(block_of_target))]
        call = dict(indices=token_to_slot, metadata=self._runtime_metadata(), scaling=1.0)
        backend = get_backend()
        if self._wants_rank_masking() and getattr(backend, "takes_effective_rank", False):
            call["effective_rank"] = self.effective_lora_rank
        if len(block_sizes) == 1:
            out_flat = backend.add_lora([out_flat], x_flat, a_slices, b_slices, **call)[0]
        else:
            blocks = list(out_flat.split(block_sizes, dim=-1))
            if block_of_target == list(range(len(block_sizes))):
                # every block has a target, in order: accumulate straight into the packed output
                backend.add_lora(blocks, x_flat, a_slices, b_slices, y_packed=out_flat, **call)
            else:
                updated = backend.add_lora([blocks[b] for b in block_of_target], x_flat, a_slices, b_slices, **call)
                for b, new_block in zip(block_of_target, updated):
                    blocks[b] = new_block
                out_flat = torch.cat(blocks, dim=-1)
        if x.ndim == 2:
            return out_flat
        return out_flat.reshape(*x.shape[:-1], out_flat.size(-1))

    def _wants_rank_masking(self) -> bool:
        """Whether the backend should be told the per-slot ranks: only buffers of more than one
        16-rank block can skip anything, and only when some resident adapter is below the padded
        rank.  A graph captured while nothing is resident must serve whatever is installed later,
        so it takes the rank-aware kernels; one captured over adapters that all fill the padded
        rank takes the plain kernels, which stay correct for later installs because an install
        zero-fills the ranks it does not use.  Decided from the host mirror only."""
        if self.max_lora_rank <= 16:
            return False
        some_resident, some_below = self._residency()
        if not some_resident:
            return _is_cuda_graph_capture()
        return some_below

    def prime_lora_cache(self) -> None:
        if not self.supports_lora:
            return
        prime = getattr(get_backend(), "prime_slice_caches", None)
        if prime is None:
            return
        n = self._num_targets()
        prime([self._a_of(p) for p in range(n)], [self._b_of(p) for p in range(n)])

    # ---- slot residency -----------------------------------------------------------------------
    def _validate_effective_rank(self, effective_rank: int) -> None:
        if effective_rank < 0 or effective_rank > self.max_lora_rank:
            raise ValueError(f"effective_rank={effective_rank} exceeds max_lora_rank={self.max_lora_rank}")

    def _validate_common_slot_payload(self, effective_rank: int, scaling: float) -> None:
        if not self.supports_lora:
            raise ValueError(f"{self.__class__.__name__} does not enable LoRA")
        if effective_rank <= 0:
            raise ValueError(f"effective_rank must be > 0, got {effective_rank}")
        if not math.isfinite(scaling):
            raise ValueError(f"LoRA scaling must be finite, got {scaling}")
        self._validate_effective_rank(effective_rank)

    def _install(self, slot_id: int, position: int, a_src: torch.Tensor, b_src: torch.Tensor, rank: int, scaling: float):
        """Slot ``slot_id`` of one target := adapter rows below ``rank`` (B pre-scaled), zero above."""
        a_dst, b_dst = self._a_of(position), self._b_of(position).data
        a_dst = a_dst.data if isinstance(a_dst, nn.Parameter) else a_dst.detach()
        if a_dst.is_cuda:
            a_src = a_src.to(a_dst.device, non_blocking=True)
            b_src = b_src.to(b_dst.device, non_blocking=True)
            if a_src.stride(-1) != 1:
                a_src = a_src.contiguous()
            if b_src.stride(-1) != 1:
                b_src = b_src.contiguous()
            _hip.install_slot(a_dst, b_dst, slot_id, a_src, b_src, rank, float(scaling))
            return
        # modules kept on the host (unit tests with a stand-in backend)
        a_dst[slot_id].zero_()
        b_dst[slot_id].zero_()
        a_dst[slot_id, :rank].copy_(a_src[:rank])
        b_dst[slot_id, :, :rank].copy_(b_src[:, :rank] * scaling)

    def _record_slot(self, slot_id: int, effective_rank: int, scaling: float) -> None:
        # The device buffers follow the host mirrors; an element is rewritten (one small launch
        # each) only when it changes, and adapters that replace each other in a slot mostly share
        # rank and scaling.
        if self._effective_lora_rank_values[slot_id] != effective_rank:
            self.effective_lora_rank[slot_id] = effective_rank
            self._effective_lora_rank_values[slot_id] = effective_rank
        if self._lora_scaling_values[slot_id] != scaling:
            self.lora_scaling[slot_id] = scaling
            self._lora_scaling_values[slot_id] = scaling
        if self._lora_base_scaling_values[slot_id] != scaling:
            self.lora_base_scaling[slot_id] = scaling
            self._lora_base_scaling_values[slot_id] = scaling

    def set_slot_lora(self, slot_id: int, lora_a, lora_b, effective_rank: int, scaling: float) -> None:
        """Make slot ``slot_id`` hold this adapter.  Multi-target layers take ``lora_a`` as
        [targets, >=rank, in] and ``lora_b`` as a list ordered like ``lora_targets``."""
        self._validate_effective_rank(effective_rank)
        if not 0 <= slot_id < self.max_loras:
            raise IndexError(f"slot_id={slot_id} is outside the {self.max_loras} slots of this layer")
        if self._target_keys():
            given = min(len(lora_a), len(lora_b))
            for position in range(self._num_targets()):
                if position < given:
                    self._install(slot_id, position, lora_a[position], lora_b[position], effective_rank, scaling)
                else:
                    self._zero_slot(slot_id, position)
        else:
            self._install(slot_id, 0, lora_a, lora_b, effective_rank, scaling)
        self._record_slot(slot_id, effective_rank, scaling)

    def _zero_slot(self, slot_id: int, position: int) -> None:
        a = self._a_of(position)
        (a.data if isinstance(a, nn.Parameter) else a.detach())[slot_id].zero_()
        self._b_of(position).data[slot_id].zero_()

    def clear_slot_lora(self, slot_id: int) -> None:
        if not self.supports_lora:
            return
        if not 0 <= slot_id < self.max_loras:
            raise IndexError(f"slot_id={slot_id} is outside the {self.max_loras} slots of this layer")
        for position in range(self._num_targets()):
            self._zero_slot(slot_id, position)
        self._record_slot(slot_id, 0, 0.0)

    def reset_lora_parameters(self) -> None:
        if not self.supports_lora:
            return
        self.lora_A.data.zero_()
        for position in range(self._num_targets()):
            self._b_of(position).data.zero_()

    def validate_slot_lora_payload(self, lora_a, lora_b, effective_rank: int, scaling: float) -> None:
        raise NotImplementedError

    # shared shape checks of the payload validators
    def _check_multi_payload(self, lora_a, lora_b, effective_rank: int, in_dim: int, out_dims: dict) -> None:
        cls = self.__class__.__name__
        if not isinstance(lora_b, list):
            raise ValueError(f"{cls} expects lora_b to be a list ordered as layer lora_targets")
        if lora_a.ndim != 3:
            raise ValueError(f"{cls} expects 3D lora_a, got shape={tuple(lora_a.shape)}")
        if lora_a.size(0) != len(self.lora_targets):
            raise ValueError(f"Expected {len(self.lora_targets)} LoRA A targets, got {lora_a.size(0)}")
        if lora_a.size(1) < effective_rank:
            raise ValueError(f"LoRA A rank dim {lora_a.size(1)} is smaller than effective_rank={effective_rank}")
        if lora_a.size(2) != in_dim:
            raise ValueError(f"Expected lora_a input dim {in_dim}, got {lora_a.size(2)}")
        if len(lora_b) != len(self.lora_targets):
            raise ValueError(f"Expected {len(self.lora_targets)} LoRA B tensors ordered as {self.lora_targets}")
        for target, target_b in zip(self.lora_targets, lora_b):
            label = f"Target '{target}'" if isinstance(target, str) else f"Target {target}"
            if target_b.ndim != 2:
                raise ValueError(f"{label} expects 2D lora_b, got shape={tuple(target_b.shape)}")
            if target_b.size(0) != out_dims[target]:
                raise ValueError(f"{label} expects output dim {out_dims[target]}, got {target_b.size(0)}")
            if target_b.size(1) < effective_rank:
                raise ValueError(f"{label} rank dim {target_b.size(1)} is smaller than effective_rank={effective_rank}")

    def _check_single_payload(self, lora_a, lora_b, effective_rank: int, in_dim: int, out_dim: int) -> None:
        cls = self.__class__.__name__
        if isinstance(lora_b, list):
            raise ValueError(f"{cls} expects tensor lora_b")
        if lora_a.ndim != 2:
            raise ValueError(f"{cls} expects 2D lora_a, got shape={tuple(lora_a.shape)}")
        if lora_b.ndim != 2:
            raise ValueError(f"{cls} expects 2D lora_b, got shape={tuple(lora_b.shape)}")
        if lora_a.size(0) < effective_rank:
            raise ValueError(f"LoRA A rank dim {lora_a.size(0)} is smaller than effective_rank={effective_rank}")
        if lora_a.size(1) != in_dim:
            raise ValueError(f"Expected lora_a input dim {in_dim}, got {lora_a.size(1)}")
        if lora_b.size(0) != out_dim:
            raise ValueError(f"Expected lora_b output dim {out_dim}, got {lora_b.size(0)}")
        if lora_b.size(1) < effective_rank:
            raise ValueError(f"LoRA B rank dim {lora_b.size(1)} is smaller than effective_rank={effective_rank}")


class _MultiTargetMixin:
    """Layers whose A buffers are stacked as ``lora_A[target, slot, r, in]`` and whose B
    buffers are separate parameters named ``lora_B_<target>``."""

    def _target_keys(self) -> list:
        return self.lora_targets

    def _a_of(self, position: int) -> torch.Tensor:
        return self.lora_A[position]

    def _b_of(self, position: int) -> nn.Parameter:
        return getattr(self, f"lora_B_{self.lora_targets[position]}")

    def _make_lora_b_weight_loader(self, target):
        def loader(param: nn.Parameter, loaded_weight: torch.Tensor):
            if loaded_weight.size(1) > self.max_lora_rank:
                raise ValueError(f"Loaded LoRA rank {loaded_weight.size(1)} exceeds max_lora_rank={self.max_lora_rank}")
            param.data.zero_()
            param.data[0, :, : loaded_weight.size(1)].copy_(loaded_weight.chunk(self.tp_size, 0)[self.tp_rank])

        return loader

    def _alloc_lora(self, in_dim: int, out_dim_of: dict) -> None:
        self.target_to_index = {target: idx for idx, target in enumerate(self.lora_targets)}
        if not self.supports_lora:
            return
        self.lora_A = nn.Parameter(torch.zeros(len(self.lora_targets), self.max_loras, self.max_lora_rank, in_dim))
        for target in self.lora_targets:
            b = nn.Parameter(torch.zeros(self.max_loras, out_dim_of[target], self.max_lora_rank))
            set_weight_loader(b, self._make_lora_b_weight_loader(target))
            setattr(self, f"lora_B_{target}", b)

    def load_lora_A(self, loaded_weight: torch.Tensor, target) -> None:
        """Single-adapter checkpoint path: A of one target into slot 0."""
        if target not in self.target_to_index:
            return
        self._validate_effective_rank(loaded_weight.size(0))
        position = self.target_to_index[target]
        self.lora_A.data[position, 0].zero_()
        self.lora_A.data[position, 0, : loaded_weight.size(0)].copy_(loaded_weight)
        self.effective_lora_rank[0] = loaded_weight.size(0)
        self._effective_lora_rank_values[0] = loaded_weight.size(0)


class LoRAQKVParallelLinear(_MultiTargetMixin, _LoRALayerBase):
    """Stacked q|k|v projection; output blocks [q_size, kv_size, kv_size] of this TP rank."""

    _BLOCK = {"q": 0, "k": 1, "v": 2}

    def __init__(
        self,
        hidden_size: int,
        head_size: int,
        total_num_heads: int,
        total_num_kv_heads: int,
        bias: bool = False,
        lora_targets: Optional[list[str]] = None,
        max_loras: int = 1,
        max_lora_rank: int | None = None,
        lora_domain: str = LM_LORA_DOMAIN,
    ):
        rank = max_lora_rank or 0
        targets = lora_targets or ["q", "k", "v"]
        super().__init__(max_loras, rank, rank > 0 and len(targets) > 0, lora_domain)
        self.tp_size, self.tp_rank = _get_world_size(), _get_rank()
        self.hidden_size, self.head_size = hidden_size, head_size
        self.total_num_heads, self.total_num_kv_heads = total_num_heads, total_num_kv_heads
        self.num_heads = divide(total_num_heads, self.tp_size)
        self.num_kv_heads = divide(total_num_kv_heads, self.tp_size)
        self.q_size = self.num_heads * head_size
        self.kv_size = self.num_kv_heads * head_size
        out = self.q_size + 2 * self.kv_size
        self.weight = nn.Parameter(torch.empty(out, hidden_size))
        set_weight_loader(self.weight, self._base_weight_loader)
        if bias:
            self.bias = nn.Parameter(torch.empty(out))
            set_weight_loader(self.bias, self._base_weight_loader)
        else:
            self.register_parameter("bias", None)
        self.lora_targets = targets
        self._alloc_lora(hidden_size, {"q": self.q_size, "k": self.kv_size, "v": self.kv_size})

    def _base_weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor, loaded_shard_id: ShardId | None = None):
        if loaded_shard_id is None:
            param.data.copy_(loaded_weight)
            return
        sizes = [self.q_size, self.kv_size, self.kv_size]
        block = self._BLOCK.get(loaded_shard_id, 2)
        rows = param.data.narrow(0, sum(sizes[:block]), sizes[block])
        rows.copy_(loaded_weight.chunk(self.tp_size, 0)[self.tp_rank])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        qkv = F.linear(x, self.weight, self.bias)
        blocks = [self._BLOCK[t] for t in self.lora_targets]
        return self._add_lora(x, qkv, [self.q_size, self.kv_size, self.kv_size], blocks)

    def validate_slot_lora_payload(self, lora_a, lora_b, effective_rank: int, scaling: float) -> None:
        self._validate_common_slot_payload(effective_rank, scaling)
        self._check_multi_payload(
            lora_a, lora_b, effective_rank, self.hidden_size, {"q": self.q_size, "k": self.kv_size, "v": self.kv_size}
        )


class LoRAMergedColumnParallelLinear(_MultiTargetMixin, _LoRALayerBase):
    """Several column-parallel projections sharing an input (gate|up); targets are block indices."""

    def __init__(
        self,
        input_size: int,
        output_sizes: list[int],
        bias: bool = False,
        lora_targets: Optional[list[int]] = None,
        max_loras: int = 1,
        max_lora_rank: int | None = None,
        lora_domain: str = LM_LORA_DOMAIN,
    ):
        rank = max_lora_rank or 0
        targets = lora_targets if lora_targets is not None else list(range(len(output_sizes)))
        super().__init__(max_loras, rank, rank > 0 and len(targets) > 0, lora_domain)
        self.tp_size, self.tp_rank = _get_world_size(), _get_rank()
        self.input_size, self.output_sizes = input_size, output_sizes
        self.shard_output_sizes = [s // self.tp_size for s in output_sizes]
        out = sum(output_sizes) // self.tp_size
        self.weight = nn.Parameter(torch.empty(out, input_size))
        set_weight_loader(self.weight, self._base_weight_loader)
        if bias:
            self.bias = nn.Parameter(torch.empty(out))
            set_weight_loader(self.bias, self._base_weight_loader)
        else:
            self.register_parameter("bias", None)
        self.lora_targets = targets
        self._alloc_lora(input_size, dict(enumerate(self.shard_output_sizes)))

    def _base_weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor, loaded_shard_id: ShardId | None = None):
        if loaded_shard_id is None:
            param.data.copy_(loaded_weight)
            return
        assert isinstance(loaded_shard_id, int)
        start = sum(self.shard_output_sizes[:loaded_shard_id])
        rows = param.data.narrow(0, start, self.shard_output_sizes[loaded_shard_id])
        rows.copy_(loaded_weight.chunk(self.tp_size, 0)[self.tp_rank])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = F.linear(x, self.weight, self.bias)
        return self._add_lora(x, out, list(self.shard_output_sizes), list(self.lora_targets))

    def validate_slot_lora_payload(self, lora_a, lora_b, effective_rank: int, scaling: float) -> None:
        self._validate_common_slot_payload(effective_rank, scaling)
        self._check_multi_payload(lora_a, lora_b, effective_rank, self.input_size, dict(enumerate(self.shard_output_sizes)))


class _SingleTargetMixin:
    """Layers with one target: ``lora_A [slots, r, in]`` and ``lora_B [slots, out, r]``."""

    def _a_of(self, position: int) -> torch.Tensor:
        return self.lora_A

    def _b_of(self, position: int) -> nn.Parameter:
        return self.lora_B


class LoRARowParallelLinear(_SingleTargetMixin, _LoRALayerBase):
    """Row-parallel projection (o, down): the input features are sharded, so is A's last dim;
    each rank adds its partial update before the layer's own all-reduce."""

    def __init__(
        self,
        input_size: int,
        output_size: int,
        bias: bool = False,
        max_loras: int = 1,
        max_lora_rank: int | None = None,
        lora_domain: str = LM_LORA_DOMAIN,
    ):
        rank = max_lora_rank or 0
        super().__init__(max_loras, rank, rank > 0, lora_domain)
        self.tp_size, self.tp_rank = _get_world_size(), _get_rank()
        self.input_size, self.output_size = input_size, output_size
        self.shard_input_size = divide(input_size, self.tp_size)
        self.weight = nn.Parameter(torch.empty(output_size, self.shard_input_size))
        set_weight_loader(self.weight, self._base_weight_loader)
        if bias:
            self.bias = nn.Parameter(torch.empty(output_size))
            set_weight_loader(self.bias, self._base_weight_loader)
        else:
            self.register_parameter("bias", None)
        if self.supports_lora:
            self.lora_A = nn.Parameter(torch.zeros(max_loras, rank, self.shard_input_size))
            set_weight_loader(self.lora_A, self._lora_a_weight_loader)
            self.lora_B = nn.Parameter(torch.zeros(max_loras, output_size, rank))

    def _base_weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        if param.dim() == 2:
            loaded_weight = loaded_weight.narrow(1, self.tp_rank * self.shard_input_size, self.shard_input_size)
        param.data.copy_(loaded_weight)

    def _lora_a_weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        if loaded_weight.size(0) > self.max_lora_rank:
            raise ValueError(f"Loaded LoRA rank {loaded_weight.size(0)} exceeds max_lora_rank={self.max_lora_rank}")
        shard = loaded_weight.narrow(1, self.tp_rank * self.shard_input_size, self.shard_input_size)
        param.data.zero_()
        param.data[0, : loaded_weight.size(0)].copy_(shard)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = F.linear(x, self.weight, self.bias if self.tp_rank == 0 else None)
        y = self._add_lora(x, y, [self.output_size], [0])
        if self.tp_size > 1 and dist.is_available() and dist.is_initialized():
            dist.all_reduce(y)
        return y

    def validate_slot_lora_payload(self, lora_a, lora_b, effective_rank: int, scaling: float) -> None:
        self._validate_common_slot_payload(effective_rank, scaling)
        self._check_single_payload(lora_a, lora_b, effective_rank, self.shard_input_size, self.output_size)


class LoRALinear(_SingleTargetMixin, _LoRALayerBase):
    """Plain (unsharded) linear with LoRA, used for the projection layers."""

    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = True,
        max_loras: int = 1,
        max_lora_rank: int | None = None,
        lora_domain: str = LM_LORA_DOMAIN,
    ):
        rank = max_lora_rank or 0
        super().__init__(max_loras, rank, rank > 0, lora_domain)
        self.in_features, self.out_features = in_features, out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features))
        else:
            self.register_parameter("bias", None)
        if self.supports_lora:
            self.lora_A = nn.Parameter(torch.zeros(max_loras, rank, in_features))
            self.lora_B = nn.Parameter(torch.zeros(max_loras, out_features, rank))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = F.linear(x, self.weight, self.bias)
        return self._add_lora(x, y, [self.out_features], [0])

    def validate_slot_lora_payload(self, lora_a, lora_b, effective_rank: int, scaling: float) -> None:
        self._validate_common_slot_payload(effective_rank, scaling)
        self._check_single_payload(lora_a, lora_b, effective_rank, self.in_features, self.out_features)


_LORA_MODULE_TYPES = (LoRAQKVParallelLinear, LoRAMergedColumnParallelLinear, LoRARowParallelLinear, LoRALinear)


def iter_lora_modules(model: nn.Module):
    for module in model.modules():
        if isinstance(module, _LORA_MODULE_TYPES) and module.lora_enabled:
            yield module


def get_lora_state_dict(model: nn.Module) -> dict:
    return {name: param.data.clone() for name, param in model.named_parameters() if "lora_" in name}
