"""The reference's golden vectors replayed through the HIP path (C-ABI library) on the GPU."""

import pytest
import torch

from helpers import DTYPES, load_golden, run_layer_case
from oracle import segment_meta as meta_oracle

pytestmark = pytest.mark.gpu

LAYERS = load_golden("layers.json")
META = load_golden("meta.json")


def _hip_backend():
    from nanovllm_voxcpm_amd.lora import HipLoRABackend, get_backend

    backend = get_backend()
    assert isinstance(backend, HipLoRABackend), backend.availability()
    return backend


@pytest.mark.parametrize("case", LAYERS["cases"], ids=lambda c: c["name"])
def test_layer_golden_vectors_hip(case):
    from nanovllm_voxcpm_amd.utils.context import reset_lora_context

    _hip_backend()
    print(f"case={case['name']}", flush=True)
    layer, x, y = run_layer_case(case, "cuda")
    expected = torch.tensor(case["expected"], dtype=DTYPES[case["dtype"]])
    assert torch.equal(y.cpu(), expected), f"{case['name']}: {y.tolist()}"
    if "expected_without_context" in case:
        reset_lora_context()
        with torch.no_grad():
            y_base = layer(x)
        assert torch.equal(y_base.cpu(), torch.tensor(case["expected_without_context"], dtype=y.dtype))


@pytest.mark.parametrize("case", LAYERS["backend_cases"], ids=lambda c: c["name"])
def test_backend_golden_vectors_hip(case):
    from nanovllm_voxcpm_amd.lora import LoRAMetadata

    backend = _hip_backend()
    dt = DTYPES[case["dtype"]]
    mk = lambda v: torch.tensor(v, dtype=dt, device="cuda")  # noqa: E731
    x = mk(case["x"])
    y = [mk(v).reshape(x.size(0), -1) for v in case["y_slices"]]
    before = [t.clone() for t in y]
    a = [mk(v) for v in case["lora_a_slices"]]
    b = [mk(v) for v in case["lora_b_slices"]]
    slots = case["token_to_slot"]
    sorted_idx, active, counts, offsets = meta_oracle.engine_layout(slots)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")  # noqa: E731
    metadata = LoRAMetadata(
        token_to_slot=i32(slots), token_indices_sorted_by_slot=i32(sorted_idx), active_slot_ids=i32(active),
        num_tokens_per_slot=i32(counts), slot_start_offsets=i32(offsets), no_lora_flag=False, num_active_loras=len(active),
    )
    # indices arrive as int64 in the reference's tests while the metadata is int32
    outs = backend.add_lora(y, x, a, b, indices=torch.tensor(slots, dtype=torch.long, device="cuda"), metadata=metadata, scaling=case["scaling"])
    for out, exp in zip(outs, case["expected"]):
        assert torch.equal(out.cpu(), torch.tensor(exp, dtype=dt).reshape(out.shape))
    if len(y) > 1:  # several slices without y_packed: the caller's tensors stay untouched
        for t, t0 in zip(y, before):
            assert torch.equal(t, t0)


def test_mismatched_token_to_slot_length_raises_before_launch():
    """reference tests/unit/test_lora_cuda.py:192-221"""
    from nanovllm_voxcpm_amd.layers.lora import LoRALinear
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, set_lora_context

    layer = LoRALinear(in_features=2, out_features=1, bias=False, max_loras=1, max_lora_rank=1).cuda()
    with torch.no_grad():
        layer.weight.zero_()
        layer.set_slot_lora(0, torch.tensor([[1.0, 0.0]], device="cuda"), torch.tensor([[2.0]], device="cuda"), 1, 1.0)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")  # noqa: E731
    set_lora_context(LoRAContext(token_to_slot=i32([0, 0, 0]), token_indices_sorted_by_slot=i32([0, 1, 2]),
                                 active_slot_ids=i32([0]), num_tokens_per_slot=i32([3]), slot_start_offsets=i32([0, 3]),
                                 no_lora_flag=False, num_active_loras=1))
    with pytest.raises(RuntimeError, match="token_to_slot length does not match flattened input rows"):
        layer(torch.tensor([[2.0, 3.0]], device="cuda"))


# ---- segment metadata built on the device -------------------------------------------------------


@pytest.mark.parametrize("case", META["engine"], ids=lambda c: str(c["token_to_slot"]))
def test_engine_layout_golden_hip(case):
    from nanovllm_voxcpm_amd.engine.lora_manager import build_lora_context_from_slot_list
    from nanovllm_voxcpm_amd.utils.context import build_lora_context_from_token_to_slot

    slots = case["token_to_slot"]
    for ctx in (
        build_lora_context_from_slot_list(slots),
        build_lora_context_from_token_to_slot(torch.tensor(slots, dtype=torch.int32, device="cuda")),
        build_lora_context_from_token_to_slot(torch.tensor(slots, dtype=torch.int64, device="cuda"), max_slots=7),
    ):
        assert ctx.no_lora_flag is False and ctx.num_active_loras == len(case["active_slot_ids"])
        assert ctx.token_to_slot.dtype == torch.int32 and ctx.token_to_slot.tolist() == slots
        assert ctx.token_indices_sorted_by_slot.tolist() == case["sorted_idx"]
        assert ctx.active_slot_ids.tolist() == case["active_slot_ids"]
        assert ctx.num_tokens_per_slot.tolist() == case["num_tokens_per_slot"]
        assert ctx.slot_start_offsets.tolist() == case["slot_start_offsets"]


@pytest.mark.parametrize("case", META["kernel_meta"], ids=lambda c: f"{c['token_to_slot']}-{c['captured_lora_counts']}")
def test_kernel_meta_golden_hip(case):
    from nanovllm_voxcpm_amd.lora_ops import LoRAKernelMeta

    meta = LoRAKernelMeta.make(case["max_loras"], 16, "cuda", captured_lora_counts=case["captured_lora_counts"])
    meta.prepare_tensors(torch.tensor(case["token_to_slot"], dtype=torch.int32, device="cuda"))
    assert meta.no_lora_flag is case["no_lora_flag"]
    assert meta.num_active_loras == case["num_active_loras"]
    if "num_tokens_per_lora_prefix" in case:
        n = len(case["num_tokens_per_lora_prefix"])
        assert meta.num_tokens_per_lora[:n].tolist() == case["num_tokens_per_lora_prefix"]
        assert meta.lora_token_start_loc[: n + 1].tolist() == case["lora_token_start_loc_prefix"]
        assert meta.active_lora_ids[:n].tolist() == case["active_lora_ids_prefix"]
        if case["sorted_idx"] is not None:
            t = len(case["token_to_slot"])
            assert meta.token_indices_sorted_by_lora_ids[:t].tolist() == case["sorted_idx"]
            args = meta.meta_args(t, specialize_active_lora=True)
            assert args[0].tolist() == case["token_to_slot"] and args[6] == case["num_active_loras"]
            assert meta.meta_args(t, specialize_active_lora=False)[6] == case["max_loras"] + 1


@pytest.mark.parametrize("case", META["graph"], ids=lambda c: c["source"].split(":")[1][:9])
def test_graph_buffers_golden_hip(case):
    from nanovllm_voxcpm_amd.engine.graph_meta import copy_lora_domain_to_graph_vars, make_graph_domain_buffers
    from nanovllm_voxcpm_amd.utils.context import LoRAContext

    bufs = make_graph_domain_buffers(case["max_rows"], case["max_lora_buckets"], "cuda")
    # start from a dirty state so that stale values cannot pass for refreshed ones
    bufs["token_to_slot"].fill_(0)
    bufs["num_tokens_per_slot"].fill_(9)
    bufs["slot_start_offsets"].fill_(9)
    tts = case["token_to_slot"]
    ctx = LoRAContext(
        token_to_slot=None if tts is None else torch.tensor(tts, dtype=torch.int32, device="cuda"),
        no_lora_flag=case["no_lora_flag"],
    )
    copy_lora_domain_to_graph_vars(bufs, ctx)
    want = meta_oracle.graph_layout(tts, case["no_lora_flag"], case["max_rows"], case["max_lora_buckets"])
    for key, exp in case["expect"].items():
        assert bufs[key].tolist() == exp, key
    for key in ("token_to_slot", "token_indices_sorted_by_slot", "active_slot_ids", "num_tokens_per_slot", "slot_start_offsets"):
        assert bufs[key].tolist() == want[key], key
