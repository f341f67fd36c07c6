"""GPU tests of per-adapter rank masking, of where segment plans are kept, and of the benchmark
configurations at their own shapes (runs on the GPU box).

Tolerances as in test_gpu_parity.py: bf16 outputs to rtol 1e-2 / atol 1e-3 against an fp64
evaluation and to about one output ulp; integer outputs bit-exact.
"""

import pytest
import torch

from test_gpu_parity import ATOL, RTOL, _apply, _backend, _check, _exact, _knobs, _make, _metadata

pytestmark = pytest.mark.gpu


# ---- per-adapter rank masking --------------------------------------------------------------------


def _poisoned(proj, ranks):
    """Copies of the projection's buffers with NaN wherever a slot's own rank ends: rows of A and
    columns of B at or above it.  Correct only for a kernel that neither reads nor multiplies them."""
    a = [t.clone() for t in proj.a]
    b = [t.clone() for t in proj.b]
    for s, r in enumerate(ranks):
        for t in a:
            t[s, r:] = float("nan")
        for t in b:
            t[s, :, r:] = float("nan")
    return a, b


@pytest.mark.parametrize("form", ["auto", "split", "mfma", "slot", "sgmv", "wide", "token"])
@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
@pytest.mark.parametrize("tokens", [200, 3000])
def test_rank_masking_never_touches_what_lies_beyond_a_slots_rank(name, tokens, form):
    """Rank-64 buffers holding adapters of rank 8, 12, 16, 32, 40 and 64 (and an empty slot), every
    element beyond a slot's rank set to NaN.  With the per-slot rank vector passed, all four
    projections in every kernel form give the fp64 result of the adapters at their own ranks:
    nothing beyond the rank is multiplied (a NaN times zero would still be NaN).  The vector is
    also what makes a slot of rank 0 a no-op."""
    from nanovllm_voxcpm_amd import _hip, synthetic

    if form == "split" and tokens > 256:
        pytest.skip("the split form takes decode-sized batches only (its exchange area holds ~128 rank-64 partial tiles)")
    print(f"rank masking {name} T={tokens} form={form}", flush=True)
    ranks = [8, 12, 16, 32, 40, 64, 0, 24]
    clean = _make(name, len(ranks), 64, torch.bfloat16, seed=800, true_ranks=ranks)
    a_nan, b_nan = _poisoned(clean, ranks)
    g = torch.Generator().manual_seed(801 + tokens)
    if tokens <= 256:
        slots = torch.randint(-1, len(ranks), (tokens,), generator=g, dtype=torch.int32)
        slots[:40] = 3  # several small tiles of one slot
    else:
        per_seq = torch.randint(-1, len(ranks), (24,), generator=g, dtype=torch.int32)
        lengths = torch.randint(1, 2 * tokens // 24, (24,), generator=g)
        slots = torch.repeat_interleave(per_seq, lengths)[:tokens]
        slots = torch.nn.functional.pad(slots, (0, tokens - slots.numel()), value=5)
    slots = slots.cuda()
    x, y0 = synthetic.make_activations(tokens, clean.k, sum(clean.widths), torch.bfloat16, seed=802, device="cuda")
    eff = torch.tensor(ranks, dtype=torch.int32, device="cuda")
    exact, mag = _exact(clean, x, y0, slots)

    backend = _backend(form)
    y = y0.clone()
    blocks = list(y.split(clean.widths, dim=-1))
    try:
        backend.add_lora(blocks, x, a_nan, b_nan, indices=slots, metadata=_metadata(slots), scaling=1.0,
                         y_packed=y if len(blocks) > 1 else None, effective_rank=eff)
    except RuntimeError as e:
        if form == "slot" and "slot-major form needs" in str(e):
            pytest.skip("the slot-major form refuses this shape (column ranges too wide for three slices, or K = 4096 at a rank and "
                        "width its K parts do not take), as AUTO knows: " + str(e))
        raise
    assert torch.isfinite(y.float()).all(), "a value beyond a slot's rank reached the output"
    _check(y, y0, exact, mag, slots, f"masked/{name}/T{tokens}/{form}")
    # the empty slot (rank 0) is a no-op even though its buffers are all NaN
    assert torch.equal(y[slots == 6], y0[slots == 6])
    # without the vector the same clean buffers (zero padding) give the same result
    got_plain = _apply(form, clean, x, y0.clone(), slots)
    keep = slots != 6
    assert torch.allclose(got_plain[keep].float(), y[keep].float(), rtol=RTOL, atol=ATOL)
    assert _hip.FORMS[form] >= 0


@pytest.mark.parametrize("form", ["auto", "sgmv", "wide", "fused", "mfma", "split"])
@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
def test_last_k_steps_of_every_k_part_count_for_adapters_of_every_rank(name, form):
    """x is zero except for the last 32 columns of every sixteenth of K (the last MFMA step of every
    K part and of every batch of one, however the kernel cuts K), so each of those steps is most of
    the result instead of a hundredth of it.  Adapters of rank 8..64 in rank-64 buffers, with the
    rank vector: a kernel that leaves rank blocks out takes a different path through its MFMAs for
    each number of blocks, and the result of the last MFMA on the shortest path (one block) was once
    read before the matrix pipeline had delivered it."""
    from nanovllm_voxcpm_amd import _hip

    tokens = 200
    if form == "fused" and "fused" not in _hip.FORMS:
        pytest.skip("no one-launch form in this library")
    print(f"last k-steps {name} form={form}", flush=True)
    ranks = [8, 12, 16, 32, 40, 64, 0, 24]
    clean = _make(name, len(ranks), 64, torch.bfloat16, seed=810, true_ranks=ranks)
    g = torch.Generator().manual_seed(811)
    slots = torch.randint(-1, len(ranks), (tokens,), generator=g, dtype=torch.int32)
    slots[:40] = 3
    slots = slots.cuda()
    from nanovllm_voxcpm_amd import synthetic

    x, y0 = synthetic.make_activations(tokens, clean.k, sum(clean.widths), torch.bfloat16, seed=812, device="cuda")
    keep = torch.zeros(clean.k, dtype=torch.bool, device="cuda")
    step = clean.k // 16
    for part in range(16):
        keep[(part + 1) * step - 32 : (part + 1) * step] = True
    x = x * keep
    eff = torch.tensor(ranks, dtype=torch.int32, device="cuda")
    exact, mag = _exact(clean, x, y0, slots)
    backend = _backend(form)
    for _ in range(2):
        y = y0.clone()
        blocks = list(y.split(clean.widths, dim=-1))
        backend.add_lora(blocks, x, clean.a, clean.b, indices=slots, metadata=_metadata(slots), scaling=1.0,
                         y_packed=y if len(blocks) > 1 else None, effective_rank=eff)
        _check(y, y0, exact, mag, slots, f"last-k-steps/{name}/{form}")


@pytest.mark.parametrize("form", ["auto", "mfma"])
@pytest.mark.parametrize("rank", [16, 64])
@pytest.mark.parametrize("k", [800, 1056])
def test_last_k_step_of_every_wavefront_counts_when_k_is_cut_at_run_time(k, rank, form):
    """A K for which the small-tile kernel has no instance of its own: its eight wavefronts share
    out the 32-column steps at run time (25 steps: 3, 3, ... 4; 33 steps: 4, 4, ... 5) and skip the
    steps past their share by branches, so the last MFMA of a wavefront may be followed by a
    branch.  x is zero except in the last step of every wavefront's share."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"last k-step per wavefront K={k} r={rank} form={form}", flush=True)
    shapes = {"w": (k, [256, 72])}
    proj = synthetic.make_projection("w", 6, rank, torch.bfloat16, seed=830 + rank, device="cuda", shapes=shapes)
    slots = synthetic.decode_slots(48, 6, seed=831).cuda()
    x, y0 = synthetic.make_activations(48, k, sum(proj.widths), torch.bfloat16, seed=832, device="cuda")
    steps = k // 32
    keep = torch.zeros(k, dtype=torch.bool, device="cuda")
    for wave in range(8):
        last = (wave + 1) * steps // 8 - 1
        keep[32 * last : 32 * last + 32] = True
    x = x * keep
    exact, mag = _exact(proj, x, y0, slots)
    for _ in range(2):
        got = _apply(form, proj, x, y0.clone(), slots)
        _check(got, y0, exact, mag, slots, f"last-k-step/K{k}/r{rank}/{form}")


def test_layers_pass_their_rank_vector_to_the_backend():
    """A rank-64 layer holding adapters of rank 8 and 64: after the padded rows / columns of the
    rank-8 slot are overwritten with NaN behind the layer's back, its forward is still the fp64
    result — the layer told the backend the slot's rank (reference keeps the vector for this:
    nanovllm_voxcpm/layers/lora.py:409-417)."""
    from nanovllm_voxcpm_amd.layers.lora import LoRAMergedColumnParallelLinear
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, set_lora_context

    g = torch.Generator().manual_seed(810)
    K, N, T = 1024, 512, 96
    layer = LoRAMergedColumnParallelLinear(K, [N, N], max_loras=3, max_lora_rank=64).cuda().to(torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_((torch.randn(2 * N, K, generator=g) * 0.02).to(torch.bfloat16))
        payload = {}
        for slot, rank in ((0, 8), (1, 64)):
            a = torch.randn(2, rank, K, generator=g) * 0.05
            b = [torch.randn(N, rank, generator=g) * 0.05 for _ in range(2)]
            payload[slot] = (a, b, rank)
            layer.set_slot_lora(slot, a.cuda(), [t.cuda() for t in b], effective_rank=rank, scaling=2.0)
        layer.lora_A.data[:, 0, 8:] = float("nan")
        layer.lora_B_0.data[0, :, 8:] = float("nan")
        layer.lora_B_1.data[0, :, 8:] = float("nan")
    assert layer._wants_rank_masking()
    x = torch.randn(T, K, generator=g).to(torch.bfloat16).cuda()
    slots = torch.randint(-1, 2, (T,), generator=g, dtype=torch.int32).cuda()
    set_lora_context(LoRAContext(token_to_slot=slots, no_lora_flag=False))
    with torch.no_grad():
        y = layer(x)
        base = torch.nn.functional.linear(x, layer.weight)
    assert torch.isfinite(y.float()).all()
    want = base.double().cpu()
    xs = x.double().cpu()
    for slot, (a, b, rank) in payload.items():
        rows = torch.nonzero(slots.cpu() == slot).flatten()
        for i in range(2):
            a16 = a[i].to(torch.bfloat16).double()
            b16 = (b[i] * 2.0).to(torch.bfloat16).double()
            want[rows, i * N : (i + 1) * N] += xs[rows] @ a16.T @ b16.T
    assert torch.allclose(y.double().cpu(), want, rtol=RTOL, atol=ATOL)
    off = slots < 0
    assert torch.equal(y[off], base[off])


# ---- where segment plans are kept ------------------------------------------------------------------


def _small_case(seed=820, tokens=64, slots_n=4):
    from nanovllm_voxcpm_amd import synthetic

    proj = _make("o", slots_n, 16, torch.bfloat16, seed=seed)
    x, y0 = synthetic.make_activations(tokens, proj.k, sum(proj.widths), torch.bfloat16, seed=seed + 1, device="cuda")
    return proj, x, y0


def test_slot_vector_rewritten_in_place_under_inference_mode_is_followed():
    """Inference tensors carry no version counter, so an in-place rewrite of the slot vector cannot
    be noticed through it: with the same metadata object the second call must still follow the
    new slot ids (no plan is kept for such tensors)."""
    proj, x, y0 = _small_case()
    backend = _backend()
    g = torch.Generator().manual_seed(821)
    first = torch.randint(-1, 4, (64,), generator=g, dtype=torch.int32)
    second = torch.randint(-1, 4, (64,), generator=g, dtype=torch.int32)
    assert not torch.equal(first, second)
    with torch.inference_mode():
        slots = first.cuda()
        meta = _metadata(slots)
        outs = []
        for new in (None, second):
            if new is not None:
                slots.copy_(new.cuda())  # same tensor, same metadata object, new contents
            y = y0.clone()
            backend.add_lora([y], x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0)
            outs.append(y.clone())
    for got, ids in zip(outs, (first, second)):
        exact, mag = _exact(proj, x, y0, ids.cuda())
        _check(got, y0, exact, mag, ids.cuda(), "in-place rewrite")


def test_context_plans_follow_an_in_place_refresh_of_graph_buffers():
    """The engine's graph path keeps one set of buffers and refreshes them in place before every
    replay.  A layer forward run eagerly on such a context must follow the refreshed slot ids: the
    refresh drops what the installed context derived from the old contents."""
    from nanovllm_voxcpm_amd.engine.graph_meta import copy_lora_domain_to_graph_vars, make_graph_domain_buffers
    from nanovllm_voxcpm_amd.layers.lora import LoRALinear
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, get_lora_context, set_lora_context

    g = torch.Generator().manual_seed(830)
    T, L = 48, 4
    layer = LoRALinear(256, 128, bias=False, max_loras=L, max_lora_rank=16).cuda().to(torch.bfloat16)
    with torch.no_grad():
        layer.weight.zero_()
        for s in range(L):
            layer.set_slot_lora(s, (torch.randn(16, 256, generator=g) * 0.1).cuda(), (torch.randn(128, 16, generator=g) * 0.1).cuda(), 16, 1.0)
    x = torch.randn(T, 256, generator=g).to(torch.bfloat16).cuda()
    bufs = make_graph_domain_buffers(T, L + 1, "cuda")
    view = LoRAContext(token_to_slot=bufs["token_to_slot"][:T], active_slot_ids=bufs["active_slot_ids"], no_lora_flag=False)
    set_lora_context(view)
    results = []
    with torch.inference_mode():
        for step in range(3):
            ids = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32).cuda()
            copy_lora_domain_to_graph_vars(bufs, LoRAContext(token_to_slot=ids, no_lora_flag=False))
            assert get_lora_context() is view and not view._segment_plans  # derived state was dropped
            y = layer(x)
            assert len(view._segment_plans) == 1  # and rebuilt once, on the context itself
            y_again = layer(x)
            assert len(view._segment_plans) == 1
            assert torch.equal(y, y_again)
            results.append((ids, y))
    a, b = layer.lora_A.detach().double().cpu(), layer.lora_B.detach().double().cpu()
    for ids, y in results:
        want = torch.zeros(T, 128, dtype=torch.float64)
        for t, s in enumerate(ids.tolist()):
            if s >= 0:
                want[t] = x[t].double().cpu() @ a[s].T @ b[s].T
        assert torch.allclose(y.double().cpu(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("form", ["mfma", "slot", "split", "sgmv", "wide", "fused", "bgmv"])
def test_a_plan_of_another_batch_shape_is_counted_not_followed(form):
    """Through the C-ABI a plan built for another (num_tokens, max_slots) is only recognised on the
    device: the call returns 0, y keeps its bits, and the launch is counted in the header of the
    plan that was passed (MLORA_PLAN_REJECTED), where a native caller can see it.  The matching
    plan, passed next, is followed and not counted."""
    from nanovllm_voxcpm_amd import _hip, synthetic
    from nanovllm_voxcpm_amd.lora_ops import build_segment_plan

    T, L = 200, 8
    proj = _make("o", L, 16, torch.bfloat16, seed=870)
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=871, device="cuda")
    g = torch.Generator().manual_seed(872)
    slots = torch.randint(0, L, (T,), generator=g, dtype=torch.int32).cuda()
    longer = torch.randint(0, L, (2 * T,), generator=g, dtype=torch.int32).cuda()
    stale = build_segment_plan(longer, L)        # built for 400 tokens: larger than any offset a call for 200 reads
    other_slots = build_segment_plan(torch.cat([slots, slots]), L + 8)
    good = build_segment_plan(slots, L)
    scratch = torch.empty(_hip.add_workspace_bytes(T, 1, 16, torch.bfloat16), dtype=torch.uint8, device="cuda")
    _hip.workspace_init(scratch)
    print(f"stale plan, form {form}", flush=True)
    for plan in (stale, other_slots):
        y = y0.clone()
        _hip.add_lora(y, x, proj.a, proj.b, [0], slots, plan.workspace, 1.0, _hip.FORMS[form], scratch)
        torch.cuda.synchronize()
        assert torch.equal(y, y0), "a plan of another batch shape was followed"
        assert plan.rejected_launches() >= 1
    y = y0.clone()
    _hip.add_lora(y, x, proj.a, proj.b, [0], slots, good.workspace, 1.0, _hip.FORMS[form], scratch)
    exact, mag = _exact(proj, x, y0, slots)
    _check(y, y0, exact, mag, slots, f"matching plan/{form}")
    assert good.rejected_launches() == 0


def test_context_plans_follow_a_versioned_slot_vector_rewritten_in_place():
    """A context that lives across steps and whose slot vector is rewritten with ``copy_`` outside
    inference mode (nobody announces the write): the tensor's version counter is part of the key of
    the context's plan table, so the next forward builds a new plan and follows the new slot ids.
    A new vector put on the same context without installing it again is followed too."""
    from nanovllm_voxcpm_amd.layers.lora import LoRALinear
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, reset_lora_context, set_lora_context

    g = torch.Generator().manual_seed(835)
    T, L = 48, 4
    layer = LoRALinear(256, 128, bias=False, max_loras=L, max_lora_rank=16).cuda().to(torch.bfloat16)
    with torch.no_grad():
        layer.weight.zero_()
        for s in range(L):
            layer.set_slot_lora(s, (torch.randn(16, 256, generator=g) * 0.1).cuda(), (torch.randn(128, 16, generator=g) * 0.1).cuda(), 16, 1.0)
    x = torch.randn(T, 256, generator=g).to(torch.bfloat16).cuda()
    a, b = layer.lora_A.detach().double().cpu(), layer.lora_B.detach().double().cpu()

    def want_for(ids):
        want = torch.zeros(T, 128, dtype=torch.float64)
        for t, s in enumerate(ids.tolist()):
            if s >= 0:
                want[t] = x[t].double().cpu() @ a[s].T @ b[s].T
        return want

    first = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32)
    second = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32)
    third = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32)
    assert not torch.equal(first, second) and not torch.equal(second, third)
    slots = first.cuda()
    ctx = LoRAContext(token_to_slot=slots, no_lora_flag=False)
    set_lora_context(ctx)
    try:
        with torch.no_grad():
            y1 = layer(x)
            slots.copy_(second.cuda())  # same tensor, same context, new contents, no announcement
            y2 = layer(x)
            y2_again = layer(x)
            ctx.token_to_slot = third.cuda()  # a new vector on the same, still installed context
            y3 = layer(x)
    finally:
        reset_lora_context()
    assert torch.equal(y2, y2_again)
    for got, ids in ((y1, first), (y2, second), (y3, third)):
        assert torch.allclose(got.double().cpu(), want_for(ids), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("name,tokens,rank", [("down", 200, 16), ("gate_up", 2000, 64)])
def test_two_streams_share_one_metadata_object(name, tokens, rank):
    """A plan is read-only for the apply kernels (what workgroups exchange lives in the scratch,
    one buffer per device and stream), so two streams may run the same step's metadata at the
    same time: both results are bit-identical to a single-stream run."""
    from nanovllm_voxcpm_amd import synthetic
    from nanovllm_voxcpm_amd.lora import _PLAN_ATTR

    print(f"two streams {name} T={tokens} r={rank}", flush=True)
    proj = _make(name, 6, rank, torch.bfloat16, seed=840)
    x, y0 = synthetic.make_activations(tokens, proj.k, sum(proj.widths), torch.bfloat16, seed=841, device="cuda")
    g = torch.Generator().manual_seed(842)
    slots = torch.randint(-1, 6, (tokens,), generator=g, dtype=torch.int32)
    slots[: tokens // 3] = 1
    slots = slots.cuda()
    backend = _backend()
    meta = _metadata(slots)

    def run(y):
        blocks = list(y.split(proj.widths, dim=-1))
        backend.add_lora(blocks, x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0,
                         y_packed=y if len(blocks) > 1 else None)

    reference = y0.clone()
    run(reference)
    torch.cuda.synchronize()
    assert len(getattr(meta, _PLAN_ATTR)) == 1
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[y0.clone() for _ in range(6)] for _ in streams]
    torch.cuda.synchronize()
    for round_ in range(6):
        for s, stream in enumerate(streams):
            with torch.cuda.stream(stream):
                run(outs[s][round_])
    torch.cuda.synchronize()
    assert len(getattr(meta, _PLAN_ATTR)) == 1  # one plan served every call
    for per_stream in outs:
        for y in per_stream:
            assert torch.equal(y, reference)


# ---- benchmark configurations at their own shapes ----------------------------------------------------


@pytest.mark.parametrize("name", ["gate_up", "down"])
def test_config3_prefill_full_batch_wide_projections(name):
    """configs[2] at its own size (16 sequences of 64..1024 tokens, 8 adapters of rank 64, a quarter
    of the sequences without adapter) for the two wide projections, element by element against the
    fp64 evaluation."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"config3 full {name}", flush=True)
    proj = _make(name, 8, 64, torch.bfloat16, seed=300)
    slots_cpu, _ = synthetic.prefill_slots(16, 8, seed=301)
    T = slots_cpu.numel()
    assert T > 8000 and (slots_cpu < 0).any()
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=302, device="cuda")
    slots = slots_cpu.cuda()
    got = _apply("auto", proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, f"config3-full/{name}")


@pytest.mark.parametrize("layer", [0, 1, 2])
@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
def test_config4_mixed_batch_every_projection_three_layers(name, layer):
    """configs[3]: 8192 tokens (2 x 2048-token chunks + 4096 decodes), 128 adapters of ranks
    {8,16,32,64} in rank-64 buffers, Zipf(1.1) popularity; every projection, three independently
    seeded layers, with the per-slot rank vector passed (what the LoRA linears do for such
    buffers) and padding that would poison the result if it were read."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"config4 {name} layer {layer}", flush=True)
    ranks = synthetic.heterogeneous_ranks(128, seed=400)
    clean = _make(name, 128, 64, torch.bfloat16, seed=401 + 16 * layer, true_ranks=ranks)
    a_nan, b_nan = _poisoned(clean, ranks)
    slots_cpu = synthetic.mixed_slots(seed=402)
    assert slots_cpu.numel() == 8192
    x, y0 = synthetic.make_activations(8192, clean.k, sum(clean.widths), torch.bfloat16, seed=403 + layer, device="cuda")
    slots = slots_cpu.cuda()
    eff = torch.tensor(ranks, dtype=torch.int32, device="cuda")
    y = y0.clone()
    blocks = list(y.split(clean.widths, dim=-1))
    _backend().add_lora(blocks, x, a_nan, b_nan, indices=slots, metadata=_metadata(slots), scaling=1.0,
                        y_packed=y if len(blocks) > 1 else None, effective_rank=eff)
    exact, mag = _exact(clean, x, y0, slots)
    _check(y, y0, exact, mag, slots, f"config4/{name}/layer{layer}")


def test_config5_backbone_at_its_own_shape():
    """configs[4]: 24 layers, hidden 1024, 16 query / 2 KV heads of 64 (kv width 128), SwiGLU 4096,
    64 decode streams with context lengths U[128, 2048], 32 rank-32 adapters on all linears, bf16.
    The HIP path inside the whole decode step against the same step through the oracle backend
    (the reference's per-token torch loop), both measured against the step evaluated in fp32 on
    the same bf16-valued weights: element by element the HIP path stays within the bf16 error
    budget of 24 layers, and on average it is no further from the fp32 result than the reference
    formulation run in bf16."""
    import copy

    from nanovllm_voxcpm_amd.backbone import MiniDecoder
    from nanovllm_voxcpm_amd.lora import HipLoRABackend
    from oracle.lora_apply import OracleBackend
    from test_backbone import _run

    streams, adapters, rank = 64, 32, 32
    model = MiniDecoder(max_loras=adapters, rank=rank).to(device="cuda", dtype=torch.bfloat16)
    assert len(model.layers) == 24 and model.hidden == 1024 and model.layers[0].qkv.kv_size == 128
    model.init_random(seed=500, adapters=adapters, rank=rank)
    g = torch.Generator().manual_seed(501)
    positions = torch.randint(128, 2049, (streams,), generator=g).cuda()
    slots = torch.randint(0, adapters, (streams,), generator=g, dtype=torch.int32)
    slots[::9] = -1  # a few streams without adapter
    slots = slots.cuda()
    x = torch.randn(streams, model.hidden, generator=g).to(torch.bfloat16).cuda()
    cache = [(k.cpu(), v.cpu()) for k, v in model.make_cache(streams, 2049, torch.bfloat16, "cuda", seed=502)]

    got = _run(model, x, positions, slots, cache, HipLoRABackend(), lora=True)
    base = _run(model, x, positions, slots, cache, HipLoRABackend(), lora=False)
    ref16 = _run(model, x, positions, slots, cache, OracleBackend(), lora=True)
    model32 = copy.deepcopy(model).float()
    cache32 = [(k.float(), v.float()) for k, v in cache]
    exact = _run(model32, x.float(), positions, slots, cache32, OracleBackend(), lora=True)

    off = slots < 0
    assert torch.equal(got[off], base[off])  # streams without adapter: bit-identical to LoRA disabled
    assert ((got[~off].float() - base[~off].float()).abs().amax(dim=-1) > 1e-2).all()
    err_hip = (got.float() - exact).abs()
    err_ref = (ref16.float() - exact).abs()
    # Both bf16 runs carry the rounding noise of 24 layers of bf16 arithmetic around the LoRA calls
    # (a random walk of a few hundred roundings of 2^-9 each: a few percent of an element's scale,
    # outputs follow a final RMSNorm and have unit rms).  Element by element, on the scale of the
    # element and its row, the HIP path may not be further from the fp32 result than the
    # reference formulation's own worst element (with 1.5 x slack for the different draw of the
    # same noise), and never further than 15 %; on average it may not be worse either.
    scale = exact.abs() + exact.pow(2).mean(dim=-1, keepdim=True).sqrt()
    worst_hip, worst_ref = (err_hip / scale).max().item(), (err_ref / scale).max().item()
    print(f"backbone worst relative error: hip {worst_hip:.4f}, reference loop in bf16 {worst_ref:.4f}; "
          f"mean abs error: hip {err_hip.mean().item():.5f}, reference {err_ref.mean().item():.5f}", flush=True)
    assert worst_hip <= 1.5 * worst_ref and worst_hip <= 0.15, (worst_hip, worst_ref)
    assert err_hip.mean().item() <= 1.25 * err_ref.mean().item() + 1e-4, (err_hip.mean().item(), err_ref.mean().item())


# ---- the C++ host path of the usual call ------------------------------------------------------------


def test_the_cpp_host_path_enqueues_what_the_python_path_would(monkeypatch):
    """Steps of three layers x four projections, one metadata object per step as the engine installs
    one context per step, through a backend with the C++ host path and through one without
    (MLORA_NO_FASTCALL=1): the same bits for every output of every step.  The C++ path takes every
    call but those that bring something new - the first call of a step (its plan), the first use of
    a set of weight buffers - and passes on what the Python path has to answer: a slot vector
    rewritten in place (followed, not the old plan), a packed output with the wrong slice widths
    and an x of the wrong K (both raise the Python path's errors), a step whose flag says that no
    token has a slot (a no-op)."""
    from nanovllm_voxcpm_amd import _hip, synthetic
    from nanovllm_voxcpm_amd.lora import HipLoRABackend

    if _hip.load_fastcall() is None:
        pytest.skip("the C++ host path is not built (make -C nanovllm-voxcpm_amd/csrc fastcall)")
    print("C++ host path against the Python path", flush=True)
    L, rank, T = 8, 16, 96
    names = ["qkv", "o", "gate_up", "down"]
    layers = [{n: _make(n, L, rank, torch.bfloat16, seed=990 + 7 * i + j) for j, n in enumerate(names)} for i in range(3)]
    acts = {n: synthetic.make_activations(T, layers[0][n].k, sum(layers[0][n].widths), torch.bfloat16, seed=995 + j, device="cuda")
            for j, n in enumerate(names)}
    eff = torch.tensor([16, 8, 12, 16, 0, 16, 4, 16], dtype=torch.int32, device="cuda")
    g = torch.Generator().manual_seed(996)

    monkeypatch.setenv("MLORA_NO_FASTCALL", "1")
    plain = HipLoRABackend("auto")
    monkeypatch.delenv("MLORA_NO_FASTCALL")
    fast = HipLoRABackend("auto")
    assert plain._fastcall is None and fast._fastcall is not None

    def step(backend, slots, with_eff):
        meta = _metadata(slots)
        outs = []
        for layer in layers:
            for n in names:
                proj = layer[n]
                x, y0 = acts[n]
                y = y0.clone()
                blocks = list(y.split(proj.widths, dim=-1))
                got = backend.add_lora(blocks, x, proj.a, proj.b, indices=slots, metadata=meta, scaling=0.5,
                                       y_packed=y if len(blocks) > 1 else None, effective_rank=eff if with_eff else None)
                assert all(a.data_ptr() == b.data_ptr() for a, b in zip(got, blocks))
                outs.append(y)
        return outs

    calls = 0
    for s in range(4):
        slots = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32).cuda()
        want = step(plain, slots, with_eff=s % 2 == 1)
        got = step(fast, slots, with_eff=s % 2 == 1)
        calls += len(got)
        assert all(torch.equal(a, b) for a, b in zip(got, want)), f"step {s}"
    state = fast._fast_state()
    handled, passed_on = fast._fastcall.counters(state)
    # the very first call makes the state object and is not counted; passed on: every other weight
    # set's first call (11) and the first call of the other three steps
    assert handled + passed_on == calls - 1
    assert passed_on == 11 + 3 and handled == calls - 15

    # one metadata object, its slot vector rewritten in place between two calls: the second call follows the new ids
    proj = layers[0]["o"]
    x, y0 = acts["o"]
    slots = torch.randint(0, L, (T,), generator=g, dtype=torch.int32).cuda()
    meta = _metadata(slots)
    y1, y2 = y0.clone(), y0.clone()
    fast.add_lora([y1], x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0)
    fast.add_lora([y1.clone()], x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0)  # (taken in C++)
    slots.copy_(torch.randint(0, L, (T,), generator=g, dtype=torch.int32).cuda())
    fast.add_lora([y2], x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0)
    exact, mag = _exact(proj, x, y0, slots)
    _check(y2, y0, exact, mag, slots, "host path/slot vector rewritten in place")

    # what has to raise raises as before, whichever path saw the weights last
    with pytest.raises(ValueError):
        fast.add_lora([y0.clone()], x[:, :512], proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0)
    qkv = layers[0]["qkv"]
    xq, yq = acts["qkv"]
    with pytest.raises((ValueError, RuntimeError)):
        fast.add_lora(list(yq.clone().split([512, 512, 512], dim=-1)), xq, qkv.a, qkv.b, indices=slots, metadata=meta, scaling=1.0,
                      y_packed=yq.clone())
    # a step in which no token has a slot is a no-op
    from nanovllm_voxcpm_amd.lora import LoRAMetadata

    none = LoRAMetadata(token_to_slot=slots, token_indices_sorted_by_slot=None, active_slot_ids=None, num_tokens_per_slot=None,
                        slot_start_offsets=None, no_lora_flag=True, num_active_loras=0)
    y3 = y0.clone()
    fast.add_lora([y3], x, proj.a, proj.b, indices=slots, metadata=none, scaling=1.0)
    assert torch.equal(y3, y0)


def test_the_cpp_host_path_keeps_a_state_per_thread():
    """Two threads drive one backend, each on a stream of its own with its own batches: every
    thread has its own state object of the C++ host path (argument blocks, step, scratch buffer),
    so neither enqueues with what the other looked up.  Every output equals what a backend
    without the C++ path gives for the same inputs."""
    import threading

    from nanovllm_voxcpm_amd import _hip, synthetic
    from nanovllm_voxcpm_amd.lora import HipLoRABackend

    if _hip.load_fastcall() is None:
        pytest.skip("the C++ host path is not built (make -C nanovllm-voxcpm_amd/csrc fastcall)")
    print("C++ host path, two threads", flush=True)
    L, rank = 6, 32
    names = ["o", "down", "qkv"]
    projs = {n: _make(n, L, rank, torch.bfloat16, seed=1100 + j) for j, n in enumerate(names)}
    fast = HipLoRABackend("auto")
    results, errors = {}, []

    def worker(tag, T, seed):
        try:
            stream = torch.cuda.Stream()
            g = torch.Generator().manual_seed(seed)
            acts = {n: synthetic.make_activations(T, projs[n].k, sum(projs[n].widths), torch.bfloat16, seed=seed + j, device="cuda")
                    for j, n in enumerate(names)}
            outs = []
            torch.cuda.current_stream().synchronize()
            with torch.cuda.stream(stream):
                for step in range(6):
                    slots = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32).cuda()
                    meta = _metadata(slots)
                    for rep in range(2):  # every projection twice per step: the second call is the C++ path's
                        for n in names:
                            x, y0 = acts[n]
                            y = y0.clone()
                            blocks = list(y.split(projs[n].widths, dim=-1))
                            fast.add_lora(blocks, x, projs[n].a, projs[n].b, indices=slots, metadata=meta, scaling=1.0,
                                          y_packed=y if len(blocks) > 1 else None)
                            outs.append((n, slots, y))
                stream.synchronize()
            results[tag] = (acts, outs)
        except Exception as exc:  # noqa: BLE001 - reported by the main thread
            errors.append((tag, exc))

    threads = [threading.Thread(target=worker, args=("a", 80, 1200)), threading.Thread(target=worker, args=("b", 200, 1300))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    import os

    os.environ["MLORA_NO_FASTCALL"] = "1"
    try:
        plain = HipLoRABackend("auto")
    finally:
        del os.environ["MLORA_NO_FASTCALL"]
    assert plain._fastcall is None
    for tag, (acts, outs) in results.items():
        for n, slots, got in outs:
            x, y0 = acts[n]
            want = y0.clone()
            blocks = list(want.split(projs[n].widths, dim=-1))
            plain.add_lora(blocks, x, projs[n].a, projs[n].b, indices=slots, metadata=_metadata(slots), scaling=1.0,
                           y_packed=want if len(blocks) > 1 else None)
            assert torch.equal(got, want), (tag, n)
