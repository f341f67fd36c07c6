"""Seeded synthetic workloads of the benchmark configurations (used by bench.py and the tests).

Everything is generated on the host with ``torch.Generator().manual_seed`` so that the same
bits are produced on every machine, then moved to the requested device.  Weights are created
directly in the buffer layout of the LoRA linears: A ``[slots, r, K]``, B ``[slots, N, r]`` with
the adapter's ``alpha / r`` already folded into B.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

# K -> output column blocks of the four LoRA-wrapped projections of a decoder layer
PROJECTIONS = {
    "qkv": (1024, [1024, 256, 256]),
    "o": (1024, [1024]),
    "gate_up": (1024, [4096, 4096]),
    "down": (4096, [1024]),
}


@dataclass
class ProjectionWeights:
    name: str
    k: int
    widths: list[int]
    a: list[torch.Tensor]  # per slice [slots, r, K]
    b: list[torch.Tensor]  # per slice [slots, N_i, r]


def make_projection(
    name: str,
    num_slots: int,
    rank: int,
    dtype: torch.dtype,
    seed: int,
    device: str = "cpu",
    scale: float = 2.0,
    true_ranks: list[int] | None = None,
    shapes: dict | None = None,
) -> ProjectionWeights:
    """A, B ~ N(0, 0.02); B pre-multiplied by ``scale``; rows / columns at or above a slot's true
    rank are zero when ``true_ranks`` is given (heterogeneous ranks padded to ``rank``)."""
    k, widths = (shapes or PROJECTIONS)[name]
    g = torch.Generator().manual_seed(seed)
    a_list, b_list = [], []
    for n in widths:
        a = torch.randn(num_slots, rank, k, generator=g) * 0.02
        b = torch.randn(num_slots, n, rank, generator=g) * 0.02 * scale
        if true_ranks is not None:
            for s, r_eff in enumerate(true_ranks):
                a[s, r_eff:] = 0
                b[s, :, r_eff:] = 0
        a_list.append(a.to(dtype).to(device))
        b_list.append(b.to(dtype).to(device))
    return ProjectionWeights(name, k, list(widths), a_list, b_list)


def make_activations(num_tokens: int, k: int, n_total: int, dtype: torch.dtype, seed: int, device: str = "cpu"):
    """x ~ N(0,1) and a seeded N(0,1) "base output" y so that the accumulate is exercised."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(num_tokens, k, generator=g).to(dtype).to(device)
    y = torch.randn(num_tokens, n_total, generator=g).to(dtype).to(device)
    return x, y


def decode_slots(num_tokens: int, num_slots: int, seed: int) -> torch.Tensor:
    """One token per sequence, adapter id uniform over the slots."""
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, num_slots, (num_tokens,), generator=g, dtype=torch.int32)


def prefill_slots(num_seqs: int, num_slots: int, seed: int, min_len: int = 64, max_len: int = 1024, no_lora_fraction: float = 0.25):
    """Concatenated sequences with lengths uniform in [min_len, max_len]; one adapter per
    sequence; a fixed fraction of the sequences has no adapter (slot -1).  Returns (slots, lengths)."""
    g = torch.Generator().manual_seed(seed)
    lengths = torch.randint(min_len, max_len + 1, (num_seqs,), generator=g)
    per_seq = torch.randint(0, num_slots, (num_seqs,), generator=g, dtype=torch.int32)
    n_off = int(round(num_seqs * no_lora_fraction))
    off = torch.randperm(num_seqs, generator=g)[:n_off]
    per_seq[off] = -1
    slots = torch.repeat_interleave(per_seq, lengths)
    return slots.to(torch.int32), lengths.tolist()


def zipf_choice(n: int, size: int, exponent: float, g: torch.Generator) -> torch.Tensor:
    w = 1.0 / torch.arange(1, n + 1, dtype=torch.float64) ** exponent
    return torch.multinomial(w / w.sum(), size, replacement=True, generator=g).to(torch.int32)


def mixed_slots(seed: int, num_slots: int = 128, chunk: int = 2048, num_chunks: int = 2, num_decodes: int = 4096):
    """Chunked-prefill chunks followed by single-token decodes; adapters drawn per request from a
    Zipf(1.1) popularity over the slots.  Returns the slot vector of length
    num_chunks * chunk + num_decodes."""
    g = torch.Generator().manual_seed(seed)
    per_req = zipf_choice(num_slots, num_chunks + num_decodes, 1.1, g)
    lengths = torch.tensor([chunk] * num_chunks + [1] * num_decodes)
    return torch.repeat_interleave(per_req, lengths).to(torch.int32)


def heterogeneous_ranks(num_slots: int, seed: int, choices=(8, 16, 32, 64)) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    pick = torch.randint(0, len(choices), (num_slots,), generator=g)
    return [choices[i] for i in pick.tolist()]
