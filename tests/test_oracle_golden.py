"""Pins the CPU oracle: the reference's own golden vectors, closed forms and invariants.

Runs without a GPU.  The layers here are the package's LoRA linears on the host with the
oracle's per-token loop installed as the backend — the arrangement the reference's CPU tests
use with their fake backend.
"""

import numpy as np
import pytest
import torch

from helpers import DTYPES, load_golden, run_layer_case
from oracle import lora_apply as oracle
from oracle import segment_meta as meta_oracle

LAYERS = load_golden("layers.json")
META = load_golden("meta.json")


@pytest.fixture
def oracle_backend():
    from nanovllm_voxcpm_amd.lora import set_backend_for_testing

    set_backend_for_testing(oracle.OracleBackend())
    yield
    set_backend_for_testing(None)


@pytest.mark.parametrize("case", LAYERS["cases"], ids=lambda c: c["name"])
def test_layer_golden_vectors_through_oracle(case, oracle_backend):
    from nanovllm_voxcpm_amd.utils.context import reset_lora_context

    layer, x, y = run_layer_case(case, "cpu")
    expected = torch.tensor(case["expected"], dtype=DTYPES[case["dtype"]])
    assert torch.equal(y, expected), f"{case['name']}: {y.tolist()} != {expected.tolist()}"
    if "expected_without_context" in case:
        reset_lora_context()
        with torch.no_grad():
            y_base = layer(x)
        assert torch.equal(y_base, torch.tensor(case["expected_without_context"], dtype=y.dtype))


def _backend_case_tensors(case, device="cpu"):
    dt = DTYPES[case["dtype"]]
    mk = lambda v: torch.tensor(v, dtype=dt, device=device)  # noqa: E731
    y = [mk(v).reshape(len(case["x"]), -1) for v in case["y_slices"]]
    return mk(case["x"]), y, [mk(v) for v in case["lora_a_slices"]], [mk(v) for v in case["lora_b_slices"]]


@pytest.mark.parametrize("case", LAYERS["backend_cases"], ids=lambda c: c["name"])
def test_backend_golden_vectors_oracle(case):
    x, y, a, b = _backend_case_tensors(case)
    idx = torch.tensor(case["token_to_slot"], dtype=torch.int64)
    before = [t.clone() for t in y]
    for fn in (oracle.per_token_add_lora, oracle.fused_add_lora):
        outs = fn(y, x, a, b, indices=idx, scaling=case["scaling"])
        for out, exp in zip(outs, case["expected"]):
            exp_t = torch.tensor(exp, dtype=out.dtype).reshape(out.shape)
            assert torch.equal(out, exp_t)
    # without y_packed the caller's tensors are not mutated (reference lora.py:283-286)
    for t, t0 in zip(y, before):
        assert torch.equal(t, t0)


def test_per_token_in_place_with_y_packed():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 8, generator=g)
    a = [torch.randn(2, 4, 8, generator=g), torch.randn(2, 4, 8, generator=g)]
    b = [torch.randn(2, 6, 4, generator=g), torch.randn(2, 2, 4, generator=g)]
    packed = torch.randn(5, 8, generator=g)
    snapshot = packed.clone()
    views = list(packed.split([6, 2], dim=-1))
    idx = torch.tensor([0, 1, -1, 1, 0])
    outs = oracle.per_token_add_lora(views, x, a, b, indices=idx, scaling=1.0, y_packed=packed)
    assert outs[0].data_ptr() == views[0].data_ptr()
    assert torch.equal(packed[2], snapshot[2])  # slot -1 row untouched
    assert not torch.equal(packed[0], snapshot[0])


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_fused_matches_per_token_in_fp64(seed):
    """Two independent formulations (token loop with F.linear vs gather + bmm) agree to
    rounding in fp64 — a dropped scaling, transposed operand or wrong gather index fails."""
    g = torch.Generator().manual_seed(seed)
    T, K, r, L = 37, 24, 5, 4
    x = torch.randn(T, K, generator=g, dtype=torch.float64)
    a = [torch.randn(L, r, K, generator=g, dtype=torch.float64) for _ in range(3)]
    b = [torch.randn(L, n, r, generator=g, dtype=torch.float64) for n in (7, 3, 3)]
    y = [torch.randn(T, n, generator=g, dtype=torch.float64) for n in (7, 3, 3)]
    idx = torch.randint(-1, L, (T,), generator=g)
    loop = oracle.per_token_add_lora(y, x, a, b, indices=idx, scaling=0.75)
    fused = oracle.fused_add_lora(y, x, a, b, indices=idx, scaling=0.75, accumulate=torch.float64)
    for u, v in zip(loop, fused):
        assert torch.allclose(u, v, rtol=1e-12, atol=1e-12)
    for ai, bi in zip(a, b):
        d1 = oracle.fused_delta(x, ai, bi, idx, 0.75, torch.float64)
        d2 = oracle.grouped_delta(x, ai, bi, idx, 0.75, torch.float64)
        assert torch.allclose(d1, d2, rtol=1e-12, atol=1e-12)


def test_fused_invariants():
    g = torch.Generator().manual_seed(11)
    T, K, r, L, N = 16, 32, 8, 3, 12
    x = torch.randn(T, K, generator=g)
    a = torch.randn(L, r, K, generator=g)
    b = torch.randn(L, N, r, generator=g)
    y = torch.randn(T, N, generator=g)
    idx = torch.tensor([0, 1, 2, -1] * 4)
    (out,) = oracle.fused_add_lora([y], x, [a], [b], indices=idx, scaling=1.0)
    # slot -1 rows are bit-identical
    assert torch.equal(out[idx < 0], y[idx < 0])
    # zero A => no change at all (reference tests/unit/test_lora_layers.py:116-118)
    (same,) = oracle.fused_add_lora([y], x, [torch.zeros_like(a)], [b], indices=idx, scaling=1.0)
    assert torch.equal(same, y)
    # linear in B and in the scaling
    d1 = oracle.fused_delta(x, a, b, idx, 1.0, torch.float64)
    d2 = oracle.fused_delta(x, a, 2 * b, idx, 1.0, torch.float64)
    d3 = oracle.fused_delta(x, a, b, idx, 2.0, torch.float64)
    assert torch.allclose(d2, 2 * d1, rtol=1e-12, atol=0) and torch.allclose(d3, 2 * d1, rtol=1e-12, atol=0)
    # rank padding is inert: zero rows of A / columns of B beyond the true rank change nothing
    a_pad = torch.zeros(L, r + 4, K); a_pad[:, :r] = a
    b_pad = torch.zeros(L, N, r + 4); b_pad[:, :, :r] = b
    assert torch.allclose(oracle.fused_delta(x, a_pad, b_pad, idx, 1.0, torch.float64), d1, rtol=1e-12, atol=1e-12)
    # one-hot closed form: A picks feature j, B writes it to column c with weight w
    a1 = torch.zeros(1, 1, K); a1[0, 0, 5] = 1.0
    b1 = torch.zeros(1, N, 1); b1[0, 3, 0] = 2.5
    d = oracle.fused_delta(x, a1, b1, torch.zeros(T, dtype=torch.int64), 1.0)
    expect = torch.zeros(T, N); expect[:, 3] = 2.5 * x[:, 5]
    assert torch.allclose(d, expect, rtol=1e-6, atol=1e-6)


def test_shrink_expand_oracle_match_reference_test_formulas():
    """lora_shrink against the reference's expected-value loop (tests/unit/test_lora_cuda.py:868-870)
    and lora_expand against the fake op of tests/unit/test_lora_runtime.py:142-152."""
    g = torch.Generator().manual_seed(5)
    m, K, r = 4, 160, 8
    inputs = (torch.arange(m * K, dtype=torch.float32).reshape(m, K) / 100).to(torch.float16)
    lora_a = torch.randn(2, r, K, generator=g).to(torch.float16)
    mapping = torch.tensor([0, 1, 0, 1], dtype=torch.int32)
    got = oracle.lora_shrink(inputs, [lora_a], mapping, 0.5)[0].float()
    expected = torch.empty(m, r)
    for t, s in enumerate(mapping.tolist()):
        expected[t] = torch.matmul(inputs[t].float(), lora_a[s].float().transpose(0, 1)) * 0.5
    assert torch.allclose(got, expected, atol=5e-2, rtol=5e-2)
    # rows without a slot are zero-filled
    got2 = oracle.lora_shrink(inputs, [lora_a], torch.tensor([0, -1, 1, -1]), 1.0)[0]
    assert torch.count_nonzero(got2[1]) == 0 and torch.count_nonzero(got2[3]) == 0

    h = torch.randn(2, 3, 4, generator=g)
    b = [torch.randn(1, 5, 4, generator=g), torch.randn(1, 2, 4, generator=g)]
    out0 = torch.randn(3, 9, generator=g)
    zero = torch.zeros(3, dtype=torch.int32)
    for add in (False, True):
        got = oracle.lora_expand(h, b, out0, zero, offset_start=2, add_inputs=add)
        want = out0.clone()
        col = 2
        for i, w in enumerate(b):
            upd = torch.nn.functional.linear(h[i], w[0])
            if add:
                want[:, col : col + w.size(1)].add_(upd)
            else:
                want[:, col : col + w.size(1)].copy_(upd)
            col += w.size(1)
        assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)
        assert torch.equal(got[:, :2], out0[:, :2])


EXPAND_ORDER_CASES = [
    # (inputs h [1, 1, r], B [1, 1, r], y before, add_inputs, expected y) — all bf16 except h where noted.
    # Product 2^-8 - 2^-18 is rounded to B's type first (-> 2^-8), then added to y = 1 + 2^-7 in
    # that type: an exact tie that goes to the even neighbour 1 + 2^-6.  Adding in fp32 and
    # rounding once would stay at 1 + 2^-7.
    dict(h=[1.0, -(2.0 ** -9)], h_dtype=torch.bfloat16, b=[2.0 ** -8, 2.0 ** -9], y=1.0 + 2.0 ** -7, add=True, want=1.0 + 2.0 ** -6),
    dict(h=[1.0, -(2.0 ** -9)], h_dtype=torch.bfloat16, b=[2.0 ** -8, 2.0 ** -9], y=1.0 + 2.0 ** -7, add=False, want=2.0 ** -8),
    # fp32 intermediate with bf16 weights: the intermediate is cast to the weights' type before the
    # product (1 + 2^-8 + 2^-9 -> 1 + 2^-7), so the difference is 2^-7, not 1.5 * 2^-8.
    dict(h=[1.0 + 2.0 ** -8 + 2.0 ** -9, -1.0], h_dtype=torch.float32, b=[1.0, 1.0], y=0.0, add=False, want=2.0 ** -7),
    dict(h=[1.0 + 2.0 ** -8 + 2.0 ** -9, -1.0], h_dtype=torch.float32, b=[1.0, 1.0], y=4.0, add=True, want=4.0),  # 4 + 2^-7 rounds back to 4
]


@pytest.mark.parametrize("case", EXPAND_ORDER_CASES, ids=lambda c: f"{c['h_dtype']}-add{c['add']}")
def test_lora_expand_rounds_in_the_reference_order(case):
    """Hand-picked 16-bit values on which the reference's order of roundings
    (nanovllm_voxcpm/lora_ops/triton_ops/kernel_utils.py:219-228: cast the intermediate to the
    weights' type, accumulate in fp32, round the product to the weights' type, add to y in that
    type) gives a different bf16 result than any other order."""
    h = torch.tensor(case["h"], dtype=case["h_dtype"]).view(1, 1, -1)
    b = torch.tensor(case["b"], dtype=torch.bfloat16).view(1, 1, -1)
    y = torch.tensor([[case["y"]]], dtype=torch.bfloat16)
    assert h.double().flatten().tolist() == case["h"] and b.double().flatten().tolist() == case["b"]  # exactly representable
    got = oracle.lora_expand(h, [b], y, torch.zeros(1, dtype=torch.int32), add_inputs=case["add"])
    assert got.dtype == torch.bfloat16 and got.item() == case["want"]


# ---- segment metadata -----------------------------------------------------------------------


@pytest.mark.parametrize("case", META["engine"], ids=lambda c: str(c["token_to_slot"]))
def test_engine_layout_golden(case):
    s, a, c, o = meta_oracle.engine_layout(case["token_to_slot"])
    assert (s, a, c, o) == (case["sorted_idx"], case["active_slot_ids"], case["num_tokens_per_slot"], case["slot_start_offsets"])


@pytest.mark.parametrize("case", META["kernel_meta"], ids=lambda c: f"{c['token_to_slot']}-{c['captured_lora_counts']}")
def test_kernel_meta_layout_golden(case):
    got = meta_oracle.kernel_meta_layout(case["token_to_slot"], case["max_loras"], case["captured_lora_counts"])
    assert got["no_lora_flag"] is case["no_lora_flag"]
    assert got["num_active_loras"] == case["num_active_loras"]
    if "sorted_idx" in case:
        assert got["sorted_idx"] == case["sorted_idx"]
        n = len(case["num_tokens_per_lora_prefix"])
        assert got["num_tokens_per_lora"][:n] == case["num_tokens_per_lora_prefix"]
        assert got["lora_token_start_loc"][: n + 1] == case["lora_token_start_loc_prefix"]
        assert got["active_lora_ids"][:n] == case["active_lora_ids_prefix"]


@pytest.mark.parametrize("case", META["graph"], ids=lambda c: c["source"].split(":")[1][:9])
def test_graph_layout_golden(case):
    got = meta_oracle.graph_layout(case["token_to_slot"], case["no_lora_flag"], case["max_rows"], case["max_lora_buckets"])
    for key, want in case["expect"].items():
        assert got[key] == want, key


@pytest.mark.parametrize("seed", range(5))
def test_layouts_agree_with_brute_force_sort(seed):
    rng = np.random.default_rng(seed)
    T, L = int(rng.integers(1, 200)), int(rng.integers(1, 12))
    slots = [int(v) for v in rng.integers(-1, L, size=T)]
    s, a, c, o = meta_oracle.engine_layout(slots)
    brute = sorted((slot, t) for t, slot in enumerate(slots) if slot >= 0)
    assert s == [t for _, t in brute]
    assert a == sorted({slot for slot in slots if slot >= 0})
    assert c == [sum(1 for v in slots if v == slot) for slot in a]
    assert o == [0] + list(np.cumsum(c))
    km = meta_oracle.kernel_meta_layout(slots, L)
    if not km["no_lora_flag"]:
        assert km["sorted_idx"] == [t for _, t in sorted((slot, t) for t, slot in enumerate(slots))]
        # dropping the -1 bucket from the kernel-meta layout gives the engine layout
        n_neg = slots.count(-1)
        assert km["sorted_idx"][n_neg:] == s
    gl = meta_oracle.graph_layout(slots, False, T + 3, L + 1)
    assert gl["token_indices_sorted_by_slot"][: len(s)] == s
    assert gl["num_tokens_per_slot"][0] == 0
    assert [gl["num_tokens_per_slot"][slot + 1] for slot in a] == c
    assert gl["slot_start_offsets"][-1] == len(s)
    short, long_small, long_big = meta_oracle.plan_tiles(slots, L)
    covered = sorted(p for tiles in (short, long_small) for (_, st, n) in tiles for p in range(st, st + n))
    assert covered == list(range(len(s)))
    assert sorted(p for (_, st, n) in long_big for p in range(st, st + n)) == sorted(
        p for (_, st, n) in long_small for p in range(st, st + n)
    )
    # the list by slot holds exactly the small tiles, every position once, a slot's first tile
    # under its own id and slots without tokens with count 0 at their place in the running totals
    first, further = meta_oracle.plan_tiles_by_slot(slots, L)
    assert len(first) == L and all(0 <= cnt <= 16 for cnt, _ in first)
    assert sorted([(sl, st, cnt) for sl, (cnt, st) in enumerate(first) if cnt] + further) == sorted(short + long_small)
    for sl, (cnt, st) in enumerate(first):
        assert st == sum(1 for v in slots if 0 <= v < sl)
        assert cnt == min(16, slots.count(sl))
        assert all(slots[s[p]] == sl for p in range(st, st + cnt))
    assert all(slots[s[p]] == sl for (sl, st, cnt) in further for p in range(st, st + cnt))


def test_big_tiles_are_laid_out_in_runs_over_one_block_per_xcd():
    """Properties of the placement that do not restate its rule: no two tiles share a place, all
    places lie in the list, every block (an eighth of the list) is filled from its start, the
    blocks' tile counts differ by at most one run, a block holds whole runs of consecutive tiles
    (the last run of the batch aside), a batch of many one-tile slots is dealt out tile by tile
    (every layer of eight places holds eight consecutive tiles), and a batch of few slots with many
    tiles each lets a slot meet at most two blocks more than its share of an eighth of the tiles."""
    rng = np.random.default_rng(77)

    def check(slots, T, L):
        _, _, long_big = meta_oracle.plan_tiles(slots, L)
        n = len(long_big)
        cap = meta_oracle.big_tile_capacity(T, L)
        assert cap % 32 == 0
        place = meta_oracle.big_tile_places(long_big, T, L)
        assert len(place) == n
        if n == 0:
            return None
        assert len(set(place)) == n and min(place) >= 0 and max(place) < cap
        blk = cap // 8
        by_block = {}
        for t, q in enumerate(place):
            by_block.setdefault(q // blk, {})[q % blk] = t
        counts = []
        for x, members in by_block.items():
            assert sorted(members) == list(range(len(members)))  # filled from its start
            counts.append(len(members))
        tiles = [[members[j] for j in range(len(members))] for members in by_block.values()]
        runs = [len(r) for ts in tiles for r in np.split(np.array(ts), np.nonzero(np.diff(ts) != 1)[0] + 1)]
        run = max(runs)
        assert sum(1 for r in runs if r != run) <= 1  # whole runs, but for the last of the batch
        assert max(counts) - (min(counts) if len(counts) == 8 else 0) <= run
        return long_big, place, blk, run

    for T, L in [(64, 1), (700, 3), (9392, 8), (8192, 128), (4096, 64), (100000, 16), (300, 300)]:
        lengths = rng.integers(1, max(2, 2 * T // max(1, L)), size=L)
        slots = np.repeat(np.arange(L), lengths)[:T].tolist()
        slots += [-1] * (T - len(slots))
        check(slots, T, L)
    # many slots of one tile each: tile by tile
    slots = np.repeat(np.arange(100), 20).tolist()
    long_big, place, blk, run = check(slots, len(slots), 100)
    assert run == 1 and [q // blk for q in place[:16]] == list(range(8)) * 2
    # six slots of twenty tiles each: a slot meets few blocks
    slots = np.repeat(np.arange(6), 20 * 64).tolist()
    long_big, place, blk, run = check(slots, len(slots), 6)
    for s_ in range(6):
        assert len({place[t] // blk for t in range(len(long_big)) if long_big[t][0] == s_}) <= 20 * 8 // len(long_big) + 2
