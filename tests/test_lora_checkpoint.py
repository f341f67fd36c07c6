"""LoRA checkpoint directory -> payloads -> resident slot.  The first case and the error cases
are the reference's own fixtures (tests/unit/test_voxcpm_lora_checkpoint_loader.py:9-111), as data."""

from __future__ import annotations

import json

import pytest
import torch
import torch.nn as nn
from safetensors.torch import save_file

from oracle.lora_apply import OracleBackend


def _write(tmp_path, tensors, config=None):
    d = tmp_path / "demo_lora"
    d.mkdir()
    save_file(tensors, str(d / "lora_weights.safetensors"))
    (d / "lora_config.json").write_text(json.dumps(config if config is not None else {"lora_config": {"r": 2, "alpha": 8.0}}), encoding="utf-8")
    return d


T = torch.tensor


def test_payloads_and_tensor_parallel_shards(tmp_path):
    from nanovllm_voxcpm_amd.lora_checkpoint import load_voxcpm_lora_checkpoint

    d = _write(tmp_path, {
        "base_lm.layers.0.self_attn.q_proj.lora_A": T([[1.0, 2.0], [3.0, 4.0]]),
        "base_lm.layers.0.self_attn.q_proj.lora_B": T([[10.0, 11.0], [12.0, 13.0], [14.0, 15.0], [16.0, 17.0]]),
        "base_lm.layers.0.self_attn.v_proj.lora_A": T([[5.0, 6.0], [7.0, 8.0]]),
        "base_lm.layers.0.self_attn.v_proj.lora_B": T([[20.0, 21.0], [22.0, 23.0], [24.0, 25.0], [26.0, 27.0]]),
        "base_lm.layers.0.self_attn.o_proj.lora_A": T([[30.0, 31.0, 32.0, 33.0], [34.0, 35.0, 36.0, 37.0]]),
        "base_lm.layers.0.self_attn.o_proj.lora_B": T([[40.0, 41.0], [42.0, 43.0]]),
        "enc_to_lm_proj.lora_A": T([[50.0, 51.0], [52.0, 53.0]]),
        "enc_to_lm_proj.lora_B": T([[60.0, 61.0], [62.0, 63.0]]),
    })
    rank0, rank1 = load_voxcpm_lora_checkpoint(str(d), tp_size=2)
    assert (rank0.rank, rank0.alpha) == (2, 8.0)
    qkv0, qkv1 = (p.modules["base_lm.layers.0.self_attn.qkv_proj"] for p in (rank0, rank1))
    assert qkv0.lora_a.shape == (2, 2, 2) and [t.shape for t in qkv0.lora_b] == [(2, 2), (2, 2)]
    assert torch.equal(qkv0.lora_a, T([[[1.0, 2.0], [3.0, 4.0]], [[5.0, 6.0], [7.0, 8.0]]]))  # q then v
    assert torch.equal(qkv0.lora_b[0], T([[10.0, 11.0], [12.0, 13.0]]))
    assert torch.equal(qkv1.lora_b[0], T([[14.0, 15.0], [16.0, 17.0]]))
    assert torch.equal(qkv1.lora_b[1], T([[24.0, 25.0], [26.0, 27.0]]))
    o0, o1 = (p.modules["base_lm.layers.0.self_attn.o_proj"] for p in (rank0, rank1))
    assert torch.equal(o0.lora_a, T([[30.0, 31.0], [34.0, 35.0]])) and torch.equal(o1.lora_a, T([[32.0, 33.0], [36.0, 37.0]]))
    assert torch.equal(o0.lora_b, o1.lora_b)
    assert torch.equal(rank0.modules["enc_to_lm_proj"].lora_a, rank1.modules["enc_to_lm_proj"].lora_a)
    assert qkv0.effective_rank == 2 and qkv0.scaling == 4.0
    whole = load_voxcpm_lora_checkpoint(str(d))
    assert torch.equal(whole.modules["base_lm.layers.0.self_attn.o_proj"].lora_a, T([[30.0, 31.0, 32.0, 33.0], [34.0, 35.0, 36.0, 37.0]]))


def test_prefixes_rank_inference_and_gate_up_order(tmp_path):
    from nanovllm_voxcpm_amd.lora_checkpoint import load_voxcpm_lora_checkpoint

    d = _write(tmp_path, {
        "base_model.model.model.mlp.up_proj.lora_A": torch.full((3, 4), 2.0),
        "base_model.model.model.mlp.up_proj.lora_B": torch.full((6, 3), 3.0),
        "module.mlp.gate_proj.lora_A": torch.full((3, 4), 1.0),
        "module.mlp.gate_proj.lora_B": torch.full((6, 3), 4.0),
        "unrelated.bias": torch.zeros(2),
    }, {"lora_config": {"lora_alpha": 6}})
    p = load_voxcpm_lora_checkpoint(str(d))
    assert p.rank == 3 and p.alpha == 6.0 and list(p.modules) == ["mlp.gate_up_proj"]
    m = p.modules["mlp.gate_up_proj"]
    assert m.lora_a[0, 0, 0] == 1.0 and m.lora_a[1, 0, 0] == 2.0  # gate (0) before up (1)
    assert m.lora_b[0][0, 0] == 4.0 and m.lora_b[1][0, 0] == 3.0 and m.scaling == 2.0


@pytest.mark.parametrize("tensors,config,err,text", [
    ({}, {"alpha": 8}, ValueError, "lora_config"),
    ({"a.q_proj.lora_A.weight": torch.ones(2, 2), "a.q_proj.lora_B.weight": torch.ones(2, 2)}, None, ValueError, "Unsupported LoRA tensor suffix"),
    ({"a.q_proj.lora_A": torch.ones(2, 2), "a.q_proj.lora_B": torch.ones(2, 2), "a.v_proj.lora_A.weight": torch.ones(2, 2)}, None,
     ValueError, "Unsupported LoRA tensor suffix"),
    ({"a.q_proj.lora_A": torch.ones(2, 2)}, None, ValueError, "Incomplete LoRA tensors"),
    ({"x.bias": torch.ones(2)}, None, ValueError, "does not contain any supported module"),
    ({"a.o_proj.lora_A": torch.ones(2, 2), "a.o_proj.lora_B": torch.ones(2, 2)}, {"lora_config": {"r": 3, "alpha": 1}}, ValueError, "does not match tensor rank"),
    ({"a.o_proj.lora_A": torch.ones(2, 2), "a.o_proj.lora_B": torch.ones(2, 2), "b.o_proj.lora_A": torch.ones(3, 2), "b.o_proj.lora_B": torch.ones(2, 3)},
     {"lora_config": {"alpha": 1}}, ValueError, "inconsistent ranks"),
    ({"a.o_proj.lora_A": torch.ones(2, 2), "a.o_proj.lora_B": torch.ones(2, 2)}, {"lora_config": {"r": 2}}, ValueError, "alpha or lora_alpha"),
    ({"a.o_proj.lora_A": torch.ones(2, 2), "a.o_proj.lora_B": torch.ones(2, 2)}, {"lora_config": {"r": 2, "alpha": 0}}, ValueError, "alpha must be > 0"),
])
def test_rejected_checkpoints(tmp_path, tensors, config, err, text):
    from nanovllm_voxcpm_amd.lora_checkpoint import load_voxcpm_lora_checkpoint

    with pytest.raises(err, match=text):
        load_voxcpm_lora_checkpoint(str(_write(tmp_path, tensors, config)))


def test_missing_files(tmp_path):
    from nanovllm_voxcpm_amd.lora_checkpoint import load_voxcpm_lora_checkpoint

    with pytest.raises(FileNotFoundError, match="directory not found"):
        load_voxcpm_lora_checkpoint(str(tmp_path / "nope"))
    (tmp_path / "half").mkdir()
    with pytest.raises(FileNotFoundError, match="Missing LoRA weights file"):
        load_voxcpm_lora_checkpoint(str(tmp_path / "half"))


class _Block(nn.Module):
    def __init__(self):
        super().__init__()
        from nanovllm_voxcpm_amd.layers.lora import LoRAMergedColumnParallelLinear, LoRAQKVParallelLinear, LoRARowParallelLinear

        kw = dict(max_loras=2, max_lora_rank=4)
        self.qkv_proj = LoRAQKVParallelLinear(8, 4, 2, 1, **kw)
        self.o_proj = LoRARowParallelLinear(8, 8, **kw)
        self.gate_up_proj = LoRAMergedColumnParallelLinear(8, [12, 12], **kw)
        self.plain = nn.Linear(8, 8)


def test_checkpoint_to_resident_slot_to_forward(tmp_path):
    """Disk -> payload -> install into slot 1 -> layer forward (oracle backend on the host) equals
    x W^T + (alpha / r) (x A^T) B^T; a second install into the same slot replaces the first and
    clears the module the new adapter does not touch."""
    from nanovllm_voxcpm_amd.lora import set_backend_for_testing
    from nanovllm_voxcpm_amd.lora_checkpoint import install_lora_payload, load_voxcpm_lora_checkpoint
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, reset_lora_context, set_lora_context

    g = torch.Generator().manual_seed(3)
    r = 2
    model = nn.ModuleDict({"blk": _Block()})
    with torch.no_grad():
        for m in (model["blk"].qkv_proj, model["blk"].o_proj, model["blk"].gate_up_proj):
            m.weight.copy_(torch.randn(m.weight.shape, generator=g) * 0.2)
    rnd = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    tensors = {
        "blk.q_proj.lora_A": rnd(r, 8), "blk.q_proj.lora_B": rnd(8, r),
        "blk.k_proj.lora_A": rnd(r, 8), "blk.k_proj.lora_B": rnd(4, r),
        "blk.v_proj.lora_A": rnd(r, 8), "blk.v_proj.lora_B": rnd(4, r),
        "blk.o_proj.lora_A": rnd(r, 8), "blk.o_proj.lora_B": rnd(8, r),
    }
    first = load_voxcpm_lora_checkpoint(str(_write(tmp_path, tensors, {"lora_config": {"r": r, "alpha": 6.0}})))
    loaded: dict = {}
    install_lora_payload(model, 1, first, loaded=loaded)
    assert loaded == {1: ["blk.qkv_proj", "blk.o_proj"]}

    x = rnd(3, 8)
    set_backend_for_testing(OracleBackend())
    set_lora_context(LoRAContext(token_to_slot=T([1, -1, 1], dtype=torch.int32), no_lora_flag=False))
    try:
        with torch.no_grad():
            got_qkv, got_o = model["blk"].qkv_proj(x), model["blk"].o_proj(x)
        want = x @ model["blk"].qkv_proj.weight.T
        scale = 6.0 / r
        delta = torch.cat([(x @ tensors[f"blk.{t}_proj.lora_A"].T) @ tensors[f"blk.{t}_proj.lora_B"].T for t in "qkv"], dim=-1) * scale
        delta[1] = 0
        assert torch.allclose(got_qkv, want + delta, atol=1e-5)
        d_o = (x @ tensors["blk.o_proj.lora_A"].T) @ tensors["blk.o_proj.lora_B"].T * scale
        d_o[1] = 0
        assert torch.allclose(got_o, x @ model["blk"].o_proj.weight.T + d_o, atol=1e-5)

        second = {"blk.gate_proj.lora_A": rnd(r, 8), "blk.gate_proj.lora_B": rnd(12, r),
                  "blk.up_proj.lora_A": rnd(r, 8), "blk.up_proj.lora_B": rnd(12, r),
                  "blk.o_proj.lora_A": rnd(r, 8), "blk.o_proj.lora_B": rnd(8, r)}
        (tmp_path / "second").mkdir()
        install_lora_payload(model, 1, load_voxcpm_lora_checkpoint(str(_write(tmp_path / "second", second, {"lora_config": {"alpha": 2.0}}))), loaded=loaded)
        assert loaded == {1: ["blk.gate_up_proj", "blk.o_proj"]}
        with torch.no_grad():
            assert torch.allclose(model["blk"].qkv_proj(x), want, atol=1e-6)  # cleared
            d_o = (x @ second["blk.o_proj.lora_A"].T) @ second["blk.o_proj.lora_B"].T * (2.0 / r)
            d_o[1] = 0
            assert torch.allclose(model["blk"].o_proj(x), x @ model["blk"].o_proj.weight.T + d_o, atol=1e-5)
    finally:
        reset_lora_context()
        set_backend_for_testing(None)

    with pytest.raises(ValueError, match="Unknown LoRA target module"):
        install_lora_payload(model, 0, load_voxcpm_lora_checkpoint(str(_write(tmp_path / "second" / "demo_lora", {"zzz.o_proj.lora_A": rnd(r, 8), "zzz.o_proj.lora_B": rnd(8, r)}, {"lora_config": {"alpha": 2.0}}))))
    with pytest.raises(ValueError, match="does not support LoRA slots"):
        install_lora_payload(model, 0, load_voxcpm_lora_checkpoint(str(_write(tmp_path / "second" / "demo_lora" / "demo_lora", {"blk.plain.lora_A": rnd(r, 8), "blk.plain.lora_B": rnd(8, r)}, {"lora_config": {"alpha": 2.0}}))))


def test_mismatched_payload_is_refused_before_anything_is_written(tmp_path):
    """A checkpoint made for another hidden size: every module's payload is validated against the
    module before the first write, so the slot keeps its previous adapter."""
    from nanovllm_voxcpm_amd.lora_checkpoint import install_lora_payload, load_voxcpm_lora_checkpoint

    g = torch.Generator().manual_seed(5)
    rnd = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    model = nn.ModuleDict({"blk": _Block()})
    good = {"blk.o_proj.lora_A": rnd(2, 8), "blk.o_proj.lora_B": rnd(8, 2)}
    install_lora_payload(model, 0, load_voxcpm_lora_checkpoint(str(_write(tmp_path, good))))
    before = (model["blk"].o_proj.lora_A.detach().clone(), model["blk"].qkv_proj.lora_A.detach().clone())
    bad = {"blk.q_proj.lora_A": rnd(2, 8), "blk.q_proj.lora_B": rnd(8, 2),
           "blk.o_proj.lora_A": rnd(2, 16), "blk.o_proj.lora_B": rnd(8, 2)}  # o_proj for a model twice as wide
    (tmp_path / "bad").mkdir()
    with pytest.raises(ValueError, match="input dim 8"):
        install_lora_payload(model, 0, load_voxcpm_lora_checkpoint(str(_write(tmp_path / "bad", bad))))
    assert torch.equal(model["blk"].o_proj.lora_A.detach(), before[0]) and torch.equal(model["blk"].qkv_proj.lora_A.detach(), before[1])
    with pytest.raises(IndexError, match="outside the 2 slots"):
        install_lora_payload(model, 2, load_voxcpm_lora_checkpoint(str(tmp_path / "demo_lora")))


class _WideBlock(nn.Module):
    def __init__(self, hidden=256, heads=4, kv_heads=2, head_dim=64, inter=512, max_loras=3, rank=16):
        super().__init__()
        from nanovllm_voxcpm_amd.layers.lora import LoRAMergedColumnParallelLinear, LoRAQKVParallelLinear, LoRARowParallelLinear

        kw = dict(max_loras=max_loras, max_lora_rank=rank)
        self.qkv_proj = LoRAQKVParallelLinear(hidden, head_dim, heads, kv_heads, **kw)
        self.o_proj = LoRARowParallelLinear(heads * head_dim, hidden, **kw)
        self.gate_up_proj = LoRAMergedColumnParallelLinear(hidden, [inter, inter], **kw)
        self.down_proj = LoRARowParallelLinear(inter, hidden, **kw)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_checkpoint_to_resident_slot_to_forward_on_the_gpu(tmp_path, dtype):
    """The device leg of adapter admission: checkpoint directory -> payload packed into one pinned
    host buffer -> one copy to the device -> one install launch per target -> forward of every
    LoRA linear through the HIP kernels, against x W^T + (alpha / r) (x A^T) B^T in fp64; then a
    second adapter of lower rank replaces the first in the same slot (reference:
    nanovllm_voxcpm/models/voxcpm/lora_loader.py:27-42, 134-163, engine/model_runner.py:389-420,
    fixture shape of tests/unit/test_voxcpm_lora_checkpoint_loader.py:9-69)."""
    from nanovllm_voxcpm_amd.lora import HipLoRABackend, get_backend
    from nanovllm_voxcpm_amd.lora_checkpoint import install_lora_payload, load_voxcpm_lora_checkpoint
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, reset_lora_context, set_lora_context

    print(f"checkpoint -> slot -> forward {dtype}", flush=True)
    assert isinstance(get_backend(), HipLoRABackend)
    g = torch.Generator().manual_seed(7)
    rnd = lambda *s: torch.randn(*s, generator=g) * 0.05  # noqa: E731
    hidden, q, kv, inter = 256, 256, 128, 512
    model = nn.ModuleDict({"blk": _WideBlock()}).to(device="cuda", dtype=dtype)
    mods = {n: getattr(model["blk"], n) for n in ("qkv_proj", "o_proj", "gate_up_proj", "down_proj")}
    with torch.no_grad():
        for m in mods.values():
            m.weight.copy_((torch.randn(m.weight.shape, generator=g) * 0.05).to(dtype))

    def adapter(r):
        return {
            "blk.q_proj.lora_A": rnd(r, hidden), "blk.q_proj.lora_B": rnd(q, r),
            "blk.k_proj.lora_A": rnd(r, hidden), "blk.k_proj.lora_B": rnd(kv, r),
            "blk.v_proj.lora_A": rnd(r, hidden), "blk.v_proj.lora_B": rnd(kv, r),
            "blk.o_proj.lora_A": rnd(r, q), "blk.o_proj.lora_B": rnd(hidden, r),
            "blk.gate_proj.lora_A": rnd(r, hidden), "blk.gate_proj.lora_B": rnd(inter, r),
            "blk.up_proj.lora_A": rnd(r, hidden), "blk.up_proj.lora_B": rnd(inter, r),
            "blk.down_proj.lora_A": rnd(r, inter), "blk.down_proj.lora_B": rnd(hidden, r),
        }

    T_ = 40
    slots = torch.randint(-1, 3, (T_,), generator=g, dtype=torch.int32)
    slots[:6] = 2
    x_by_k = {hidden: torch.randn(T_, hidden, generator=g).to(dtype).cuda(), inter: torch.randn(T_, inter, generator=g).to(dtype).cuda()}
    targets = {"qkv_proj": ["q", "k", "v"], "o_proj": ["o"], "gate_up_proj": ["gate", "up"], "down_proj": ["down"]}
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-3)
    loaded: dict = {}
    for step, (r, alpha) in enumerate(((16, 32.0), (8, 4.0))):
        tensors = adapter(r)
        (tmp_path / f"a{step}").mkdir()
        payload = load_voxcpm_lora_checkpoint(str(_write(tmp_path / f"a{step}", tensors, {"lora_config": {"r": r, "alpha": alpha}})))
        assert payload.packed.is_pinned()  # one pinned buffer: a slot load is one host-to-device copy
        install_lora_payload(model, 2, payload, loaded=loaded)
        set_lora_context(LoRAContext(token_to_slot=slots.cuda(), no_lora_flag=False))
        try:
            for name, m in mods.items():
                x = x_by_k[m.weight.size(1)]
                with torch.no_grad():
                    got = m(x)
                    base = torch.nn.functional.linear(x, m.weight)  # the layer's own base product, rounded to its dtype
                want = base.double().cpu()
                rows = torch.nonzero(slots == 2).flatten()
                col = 0
                for t in targets[name]:
                    a = tensors[f"blk.{t}_proj.lora_A"].to(dtype).double()
                    b = (tensors[f"blk.{t}_proj.lora_B"] * (alpha / r)).to(dtype).double()  # alpha / r folded into B at install time
                    want[rows, col : col + b.size(0)] += x.double().cpu()[rows] @ a.T @ b.T
                    col += b.size(0)
                assert torch.allclose(got.double().cpu(), want, **tol), f"{name} step {step}"
                assert m._effective_lora_rank_values[2] == r and m.effective_lora_rank.tolist()[2] == r
                # the slot holds exactly the adapter: rows / columns beyond its rank are zero
                a_buf = m.lora_A.detach()
                assert torch.count_nonzero(a_buf[..., 2, r:, :]) == 0
        finally:
            reset_lora_context()
