"""The LoRA linears composed into a whole decode step (synthetic MiniCPM-style decoder, the shape
family of the end-to-end benchmark configuration): the HIP path against the oracle backend on the
same seeded model and inputs."""

from __future__ import annotations

import pytest
import torch

from oracle.lora_apply import OracleBackend


def _build(dtype, device, layers=2):
    from nanovllm_voxcpm_amd.backbone import MiniDecoder

    model = MiniDecoder(layers=layers, hidden=256, heads=4, kv_heads=2, head_dim=64, inter=512, max_loras=4, rank=16)
    model = model.to(device=device, dtype=dtype)
    model.init_random(seed=11, adapters=4, rank=16)
    g = torch.Generator().manual_seed(12)
    streams = 24
    positions = torch.randint(3, 40, (streams,), generator=g).to(device)
    slots = torch.randint(-1, 4, (streams,), generator=g, dtype=torch.int32).to(device)
    x = torch.randn(streams, 256, generator=g).to(dtype).to(device)
    cache_cpu = [(torch.randn(streams, 2, 40, 64, generator=g).to(dtype), torch.randn(streams, 2, 40, 64, generator=g).to(dtype))
                 for _ in range(layers)]
    return model, x, positions, slots, cache_cpu


def _run(model, x, positions, slots, cache_cpu, backend, lora: bool):
    from nanovllm_voxcpm_amd.lora import set_backend_for_testing
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, reset_lora_context, set_lora_context

    caches = [(k.clone().to(x.device), v.clone().to(x.device)) for k, v in cache_cpu]
    set_backend_for_testing(backend)
    reset_lora_context()
    if lora:
        set_lora_context(LoRAContext(token_to_slot=slots, no_lora_flag=False))
    try:
        with torch.no_grad():
            return model(x, caches, positions)
    finally:
        reset_lora_context()
        set_backend_for_testing(None)


def test_backbone_with_oracle_backend_on_host():
    """Host logic only: rows without an adapter come out exactly as with LoRA disabled (every op
    of the decoder is row-wise), rows with one do not."""
    model, x, positions, slots, cache = _build(torch.float32, "cpu")
    base = _run(model, x, positions, slots, cache, OracleBackend(), lora=False)
    with_lora = _run(model, x, positions, slots, cache, OracleBackend(), lora=True)
    off = slots < 0
    assert off.any() and (~off).any()
    assert torch.equal(with_lora[off], base[off])
    assert ((with_lora[~off] - base[~off]).abs().amax(dim=-1) > 1e-3).all()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backbone_hip_path_matches_oracle_backend(dtype):
    from nanovllm_voxcpm_amd.lora import HipLoRABackend

    print(f"backbone {dtype}", flush=True)
    model, x, positions, slots, cache = _build(dtype, "cuda")
    want = _run(model, x, positions, slots, cache, OracleBackend(), lora=True)
    got = _run(model, x, positions, slots, cache, HipLoRABackend(), lora=True)
    base = _run(model, x, positions, slots, cache, HipLoRABackend(), lora=False)
    off = (slots < 0)
    assert torch.equal(got[off], base[off])
    assert (got[~off].float() - base[~off].float()).abs().amax(dim=-1).min().item() > 1e-3
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)
    else:
        # the oracle backend's loop rounds the rank-r intermediate and the update to bf16, the HIP
        # path rounds once; after eight LoRA applications and two layers of bf16 arithmetic the
        # outputs (unit scale after the final norm) agree to a few bf16 ulps
        err = (got.float() - want.float()).abs()
        assert err.max().item() < 0.1 and err.mean().item() < 6e-3
