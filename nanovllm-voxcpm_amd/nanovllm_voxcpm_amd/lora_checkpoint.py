"""LoRA checkpoint directory -> slot payloads -> resident slot.

On-disk format and resulting payloads are the reference's
(nanovllm_voxcpm/models/voxcpm/lora_loader.py:13-281): a directory with
``lora_weights.safetensors`` (keys ``<module path>.lora_A`` ``[r, in]`` / ``.lora_B`` ``[out, r]``,
optionally prefixed ``base_model.model.`` / ``model.`` / ``module.``) and ``lora_config.json``
(``{"lora_config": {"r" | "rank": int, "alpha" | "lora_alpha": float}}``).  Projections that the
model runs as one stacked linear are packed into one module payload: ``q_proj / k_proj / v_proj``
-> ``qkv_proj`` (targets in q, k, v order), ``gate_proj / up_proj`` -> ``gate_up_proj`` (targets
0, 1); their ``lora_a`` becomes ``[targets, r, in]`` and ``lora_b`` a list.  With ``tp_size > 1`` one
payload per rank is returned: packed (column-parallel) modules shard every B along its rows,
``o_proj`` / ``down_proj`` (row-parallel) shard A along its columns, everything else is replicated.

``install_lora_payload`` is the slot-loading step of the reference's model runner
(engine/model_runner.py:389-420): clear what the slot's previous occupant populated, then one
``set_slot_lora`` (here: one fused install launch) per module of the payload.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open

from nanovllm_voxcpm_amd.engine.lora_runtime import LoRAModelPayload, LoRAModulePayload

WEIGHTS_FILE = "lora_weights.safetensors"
CONFIG_FILE = "lora_config.json"

# leaf name in the checkpoint -> (stacked module it belongs to, target inside it)
PACKED_MODULES = {
    "q_proj": ("qkv_proj", "q"),
    "k_proj": ("qkv_proj", "k"),
    "v_proj": ("qkv_proj", "v"),
    "gate_proj": ("gate_up_proj", 0),
    "up_proj": ("gate_up_proj", 1),
}
_QKV_ORDER = ("q", "k", "v")
_PREFIXES = ("base_model.model.", "model.", "module.")
_ROW_PARALLEL = ("o_proj", "down_proj")
_COLUMN_PACKED = ("qkv_proj", "gate_up_proj")


def _module_path(key: str) -> str:
    """Checkpoint key without the tensor suffix and without wrapper prefixes."""
    path = key.rsplit(".", 1)[0]
    while path.startswith(_PREFIXES):
        for prefix in _PREFIXES:
            if path.startswith(prefix):
                path = path[len(prefix):]
    return path


def _read_config(directory: Path) -> dict:
    raw = json.loads((directory / CONFIG_FILE).read_text(encoding="utf-8"))
    if not isinstance(raw, dict):
        raise ValueError("LoRA config must be a JSON object")
    config = raw.get("lora_config")
    if not isinstance(config, dict):
        raise ValueError("lora_config.json must contain a 'lora_config' object")
    return config


def _alpha_of(config: dict) -> float:
    value = config["alpha"] if "alpha" in config else config.get("lora_alpha")
    if value is None:
        raise ValueError("LoRA config must define alpha or lora_alpha")
    alpha = float(value)
    if alpha <= 0:
        raise ValueError(f"LoRA alpha must be > 0, got {alpha}")
    return alpha


def _read_tensors(directory: Path) -> dict[str, dict]:
    """{module name: {target: {"a": tensor, "b": tensor}}}, targets in order of first appearance."""
    modules: dict[str, dict] = {}
    with safe_open(str(directory / WEIGHTS_FILE), framework="pt", device="cpu") as f:
        for key in f.keys():
            if key.endswith((".lora_A.weight", ".lora_B.weight")):
                raise ValueError("Unsupported LoRA tensor suffix; expected keys ending in '.lora_A' or '.lora_B'")
            if key.endswith(".lora_A"):
                kind = "a"
            elif key.endswith(".lora_B"):
                kind = "b"
            else:
                continue
            path = _module_path(key)
            parent, _, leaf = path.rpartition(".")
            if leaf in PACKED_MODULES:
                stacked, target = PACKED_MODULES[leaf]
                name = f"{parent}.{stacked}" if parent else stacked
            else:
                name, target = path, leaf
            modules.setdefault(name, {}).setdefault(target, {})[kind] = f.get_tensor(key).to(torch.float32)
    for name, targets in modules.items():
        missing_a = [t for t, pair in targets.items() if "a" not in pair]
        missing_b = [t for t, pair in targets.items() if "b" not in pair]
        if missing_a or missing_b:
            raise ValueError(f"Incomplete LoRA tensors for module '{name}': missing_a={missing_a}, missing_b={missing_b}")
    return modules


def _rank_of(modules: dict[str, dict], config: dict) -> int:
    found = sorted({pair["a"].size(0) for targets in modules.values() for pair in targets.values()})
    if not found:
        raise ValueError("LoRA checkpoint does not contain any LoRA A tensors")
    if len(found) > 1:
        raise ValueError(f"LoRA checkpoint contains inconsistent ranks: {found}")
    declared = config["r"] if "r" in config else config.get("rank")
    if declared is None:
        return found[0]
    rank = int(declared)
    if rank <= 0:
        raise ValueError(f"LoRA rank must be > 0, got {rank}")
    if rank != found[0]:
        raise ValueError(f"LoRA config rank {rank} does not match tensor rank {found[0]}")
    return rank


def _is_packed(name: str) -> bool:
    return name.endswith(_COLUMN_PACKED)


def _module_payload(name: str, targets: dict, rank: int, alpha: float) -> LoRAModulePayload:
    scaling = alpha / rank
    if _is_packed(name):
        order = [t for t in _QKV_ORDER if t in targets] if name.endswith("qkv_proj") else sorted(targets)
        return LoRAModulePayload(lora_a=torch.stack([targets[t]["a"] for t in order]), lora_b=[targets[t]["b"] for t in order],
                                 effective_rank=rank, scaling=scaling)
    pair = next(iter(targets.values()))
    return LoRAModulePayload(lora_a=pair["a"], lora_b=pair["b"], effective_rank=rank, scaling=scaling)


def _shard(name: str, module: LoRAModulePayload, tp_rank: int, tp_size: int) -> LoRAModulePayload:
    def part(t: torch.Tensor, dim: int) -> torch.Tensor:
        return t.chunk(tp_size, dim=dim)[tp_rank].contiguous()

    a, b = module.lora_a, module.lora_b
    if _is_packed(name):
        a, b = a.clone(), [part(t, 0) for t in b]
    elif name.endswith(_ROW_PARALLEL):
        a, b = part(a, 1), b.clone()
    else:
        a, b = a.clone(), ([t.clone() for t in b] if isinstance(b, list) else b.clone())
    return LoRAModulePayload(lora_a=a, lora_b=b, effective_rank=module.effective_rank, scaling=module.scaling)


def _pinned(payload: LoRAModelPayload) -> LoRAModelPayload:
    """All tensors of the payload as views of one host buffer (``payload.packed``), pinned when a GPU
    is present: a slot load then moves the adapter with one asynchronous copy instead of one per
    tensor."""
    tensors: list[torch.Tensor] = []
    for m in payload.modules.values():
        tensors.append(m.lora_a)
        tensors.extend(m.lora_b if isinstance(m.lora_b, list) else [m.lora_b])
    if not tensors or any(t.dtype != torch.float32 for t in tensors):
        return payload
    flat = torch.empty(sum(t.numel() for t in tensors), dtype=torch.float32, pin_memory=torch.cuda.is_available())
    offset = 0

    def view_of(t: torch.Tensor) -> torch.Tensor:
        nonlocal offset
        v = flat[offset : offset + t.numel()].view(t.shape)
        v.copy_(t)
        offset += t.numel()
        return v

    modules = {
        name: LoRAModulePayload(lora_a=view_of(m.lora_a),
                                lora_b=[view_of(t) for t in m.lora_b] if isinstance(m.lora_b, list) else view_of(m.lora_b),
                                effective_rank=m.effective_rank, scaling=m.scaling)
        for name, m in payload.modules.items()
    }
    packed = LoRAModelPayload(modules=modules, rank=payload.rank, alpha=payload.alpha)
    packed.packed = flat  # type: ignore[attr-defined]
    return packed


def load_voxcpm_lora_checkpoint(path: str, *, tp_size: int = 1) -> LoRAModelPayload | list[LoRAModelPayload]:
    directory = Path(path)
    if not directory.is_dir():
        raise FileNotFoundError(f"LoRA checkpoint directory not found: {directory}")
    for label, file_name in (("weights", WEIGHTS_FILE), ("config", CONFIG_FILE)):
        if not (directory / file_name).is_file():
            raise FileNotFoundError(f"Missing LoRA {label} file: {directory / file_name}")
    config = _read_config(directory)
    alpha = _alpha_of(config)
    tensors = _read_tensors(directory)
    if not tensors:
        raise ValueError("LoRA checkpoint does not contain any supported module weights")
    rank = _rank_of(tensors, config)
    full = LoRAModelPayload(modules={name: _module_payload(name, targets, rank, alpha) for name, targets in tensors.items()},
                            rank=rank, alpha=alpha)
    if tp_size <= 1:
        return _pinned(full)
    return [
        _pinned(LoRAModelPayload(modules={name: _shard(name, m, r, tp_size) for name, m in full.modules.items()}, rank=rank, alpha=alpha))
        for r in range(tp_size)
    ]


def install_lora_payload(model: torch.nn.Module, slot_id: int, payload: LoRAModelPayload, *, loaded: dict | None = None) -> None:
    """Make slot ``slot_id`` of every module named in ``payload`` hold that adapter.

    ``loaded`` (slot id -> module names, kept by the caller across calls) limits the clearing
    of the previous occupant to the modules it actually populated; without it every
    LoRA-capable module not named in the payload is cleared."""
    every = dict(model.named_modules())  # one walk over the model per admission
    modules = {name: m for name, m in every.items() if hasattr(m, "set_slot_lora")}
    for name in payload.modules:
        if name not in every:
            raise ValueError(f"Unknown LoRA target module '{name}'")
        if name not in modules:
            raise ValueError(f"Module '{name}' does not support LoRA slots")
    # every module's payload is checked against the module before anything is written: a payload
    # for another hidden size, rank budget or TP shard must not leave a half-installed slot
    for name, m in payload.modules.items():
        modules[name].validate_slot_lora_payload(m.lora_a, m.lora_b, m.effective_rank, m.scaling)
        if not 0 <= slot_id < modules[name].max_loras:
            raise IndexError(f"slot_id={slot_id} is outside the {modules[name].max_loras} slots of '{name}'")
    previous = loaded.get(slot_id) if loaded is not None and slot_id in loaded else list(modules)
    for name in previous:
        if name not in payload.modules and name in modules:
            modules[name].clear_slot_lora(slot_id)
    staged: dict = {}  # device -> copy of the payload's packed host buffer

    for name, m in payload.modules.items():
        device = next(modules[name].parameters()).device

        def put(t: torch.Tensor) -> torch.Tensor:
            packed = getattr(payload, "packed", None)
            if packed is not None and device.type == "cuda" and t.is_contiguous():
                first = (t.data_ptr() - packed.data_ptr()) // packed.element_size()
                if t.dtype == packed.dtype and 0 <= first and first + t.numel() <= packed.numel():
                    if device not in staged:
                        staged[device] = packed.to(device=device, non_blocking=True)
                    return staged[device][first : first + t.numel()].view(t.shape)
            return t.to(device=device, non_blocking=True)

        modules[name].set_slot_lora(slot_id=slot_id, lora_a=put(m.lora_a),
                                    lora_b=[put(t) for t in m.lora_b] if isinstance(m.lora_b, list) else put(m.lora_b),
                                    effective_rank=m.effective_rank, scaling=m.scaling)
    if loaded is not None:
        loaded[slot_id] = list(payload.modules)
