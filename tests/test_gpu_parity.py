"""Parity of the HIP path against the CPU oracle on seeded inputs (runs on the GPU box).

Every compute call goes through the C-ABI library via the package's backend.  Tolerances:
integer outputs (segment metadata, plans) are compared bit-exactly; bf16 / fp16 outputs are
held to rtol 1e-2 / atol 1e-3 against the reference's torch computation and, more tightly, to
about one output ulp against an fp64 evaluation of y + delta.
"""

import numpy as np
import pytest
import torch

from oracle import lora_apply as oracle
from oracle import segment_meta as meta_oracle

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3  # stated for bf16 outputs with fp32 accumulation


def _knobs(monkeypatch, **env):
    """Set (or, with None, unset) diagnostic MLORA_* variables and make the library read them."""
    from nanovllm_voxcpm_amd import _hip

    for key, value in env.items():
        if value is None:
            monkeypatch.delenv(key, raising=False)
        else:
            monkeypatch.setenv(key, str(value))
    _hip.reload_knobs()


def _waits_run_out(backend) -> int:
    """Waits of the split form that ran out, summed over the backend's scratch buffers."""
    from nanovllm_voxcpm_amd import _hip

    torch.cuda.synchronize()
    return sum(int(buf[: 4 * (_hip.WORKSPACE_TIMEOUTS_WORD + 1)].view(torch.int32)[_hip.WORKSPACE_TIMEOUTS_WORD].item())
               for buf in backend.scratch_buffers())


def _backend(form="auto"):
    from nanovllm_voxcpm_amd.lora import HipLoRABackend

    backend = HipLoRABackend(form)
    assert backend.availability().available, backend.availability().reason
    return backend


def _metadata(slots_dev):
    from nanovllm_voxcpm_amd.lora import LoRAMetadata

    return LoRAMetadata(token_to_slot=slots_dev, token_indices_sorted_by_slot=None, active_slot_ids=None,
                        num_tokens_per_slot=None, slot_start_offsets=None, no_lora_flag=False, num_active_loras=0)


def _apply(form, proj, x, y, slots, scaling=1.0):
    """Run the fused apply on the GPU for all slices of a projection; returns y (updated in place)."""
    backend = _backend(form)
    blocks = list(y.split(proj.widths, dim=-1))
    backend.add_lora(blocks, x, proj.a, proj.b, indices=slots, metadata=_metadata(slots), scaling=scaling,
                     y_packed=y if len(blocks) > 1 else None)
    return y


def _exact(proj, x, y0, slots, scaling=1.0):
    """fp64 evaluation, per slice concatenated, of y0 + delta and of sum_j |h_j| |B_nj| (the scale
    of the error a rounding of the rank-r intermediate to operand precision can cause)."""
    xs, ys, idx = x.cpu().double(), y0.cpu(), slots.cpu().to(torch.int64)
    outs, mags, col = [], [], 0
    for a, b, n in zip(proj.a, proj.b, proj.widths):
        a64, b64 = a.cpu().double(), b.cpu().double()
        d = torch.zeros(xs.size(0), n, dtype=torch.float64)
        mag = torch.zeros_like(d)
        for slot in torch.unique(idx[idx >= 0]).tolist():
            rows = torch.nonzero(idx == slot).flatten()
            h = xs[rows] @ a64[slot].T * scaling
            d[rows] = h @ b64[slot].T
            mag[rows] = h.abs() @ b64[slot].abs().T
        outs.append(ys[:, col : col + n].double() + d)
        mags.append(mag)
        col += n
    return torch.cat(outs, dim=-1), torch.cat(mags, dim=-1)


def _check(got, y0, exact, mag, slots, tag):
    got_c, y0_c = got.cpu(), y0.cpu()
    live = (slots.cpu() >= 0)
    # rows without a slot keep their bits
    assert torch.equal(got_c[~live], y0_c[~live]), f"{tag}: slot -1 rows were modified"
    want = exact.to(got.dtype)
    ok = torch.isclose(got_c.double(), want.double(), rtol=RTOL, atol=ATOL)
    assert ok.all(), f"{tag}: {(~ok).sum().item()} elements outside rtol={RTOL}/atol={ATOL}; max abs err {(got_c.double() - want.double()).abs().max().item():.4g}"
    # tighter: one rounding of the exact sum (half an ulp of the output) plus, at most, a rounding of
    # the rank-r intermediate to operand precision (MFMA forms) and fp32 accumulation noise
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -22}[got.dtype]
    bound = eps * exact.abs() + eps * mag + 2.0 ** -24
    err = (got_c.double() - exact).abs()
    bad = err > bound
    assert not bad.any(), f"{tag}: {bad.sum().item()} elements beyond one rounding; worst ratio {(err / bound).max().item():.3f}"


def _make(name, slots_n, rank, dtype, seed, **kw):
    from nanovllm_voxcpm_amd import synthetic

    return synthetic.make_projection(name, slots_n, rank, dtype, seed, device="cuda", **kw)


# ---- config 1: the reference's CPU-runnable case ------------------------------------------------


def test_config1_fp32_matches_reference_torch_loop():
    from nanovllm_voxcpm_amd import synthetic

    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 1024, generator=g)
    a_cfg = torch.randn(4, 1024, 16, generator=g) * 0.02  # config layout [L, K, r]
    b_cfg = torch.randn(4, 16, 1024, generator=g) * 0.02  # config layout [L, r, N]
    slots = torch.randint(0, 4, (64,), generator=g, dtype=torch.int32)
    a = a_cfg.transpose(1, 2).contiguous()  # buffer layout [L, r, K]
    b = b_cfg.transpose(1, 2).contiguous()  # buffer layout [L, N, r]
    y0 = torch.randn(64, 1024, generator=g)
    (want,) = oracle.per_token_add_lora([y0], x, [a], [b], indices=slots, scaling=2.0)
    y = y0.clone().cuda()
    s_dev = slots.cuda()
    _backend().add_lora([y], x.cuda(), [a.cuda()], [b.cuda()], indices=s_dev, metadata=_metadata(s_dev), scaling=2.0)
    assert torch.allclose(y.cpu(), want, rtol=1e-4, atol=1e-5)
    assert synthetic.PROJECTIONS["o"] == (1024, [1024])


# ---- config 2: decode, 256 tokens, 32 adapters of rank 16 -----------------------------------------


@pytest.mark.parametrize("form", ["auto", "bgmv", "mfma", "split", "sgmv", "wide", "token"])
@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
def test_config2_decode_bf16(name, form):
    from nanovllm_voxcpm_amd import synthetic

    print(f"config2 {name} form={form}", flush=True)
    proj = _make(name, 32, 16, torch.bfloat16, seed=100)
    x, y0 = synthetic.make_activations(256, proj.k, sum(proj.widths), torch.bfloat16, seed=101, device="cuda")
    slots = synthetic.decode_slots(256, 32, seed=102).cuda()
    got = _apply(form, proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, f"config2/{name}/{form}")


def _slot_form_batches(T, L, seed):
    """Slot vectors that exercise the slot-major grid: uniform decode ids; ids with rows without
    adapter and slot ids nobody uses; every token on one adapter (all tiles but the first are
    further tiles); a batch in which only the last slot id is used."""
    g = torch.Generator().manual_seed(seed)
    uniform = torch.randint(0, L, (T,), generator=g, dtype=torch.int32)
    sparse = torch.randint(-1, max(1, L // 2), (T,), generator=g, dtype=torch.int32)
    one = torch.full((T,), L - 1 if L > 1 else 0, dtype=torch.int32)
    one[::5] = -1
    skew = uniform.clone()
    skew[: (2 * T) // 3] = min(2, L - 1)
    return {"uniform": uniform, "sparse": sparse, "one adapter": one, "skewed": skew}


@pytest.mark.parametrize("name,rank,T,L", [("o", 16, 256, 32), ("gate_up", 16, 256, 32), ("down", 16, 256, 32), ("o", 32, 64, 32),
                                           ("gate_up", 64, 100, 5), ("o", 8, 37, 13), ("down", 8, 300, 9), ("gate_up", 32, 19, 64),
                                           ("qkv", 16, 256, 32), ("qkv", 32, 64, 32), ("qkv", 8, 37, 13), ("qkv", 64, 100, 5)])
def test_slot_major_grid_gives_the_bits_of_the_tile_major_grid(name, rank, T, L, monkeypatch):
    """The slot-major form requests a slot's weights before its record has arrived; what it computes
    is the small-tile form's arithmetic in the same order, so its results are the oracle's and,
    bit for bit, those of the tile-major grid - for slots without tokens, slot ids that are not a
    multiple of eight, rows without adapter and slots with several tiles alike."""
    from nanovllm_voxcpm_amd import synthetic

    proj = _make(name, L, rank, torch.bfloat16, seed=170 + rank)
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=171, device="cuda")
    for tag, slots in _slot_form_batches(T, L, 172 + T).items():
        print(f"slot-major {name} r={rank} T={T} L={L} {tag}", flush=True)
        slots = slots.cuda()
        got = _apply("slot", proj, x, y0.clone(), slots)
        exact, mag = _exact(proj, x, y0, slots)
        _check(got, y0, exact, mag, slots, f"slot-major/{name}/r{rank}/{tag}")
        if proj.k == 4096:  # the tile's workgroups share K out: another order of additions than one workgroup's
            _knobs(monkeypatch, MLORA_SLOT_KPARTS=1)
            assert torch.equal(_apply("slot", proj, x, y0.clone(), slots), _apply("mfma", proj, x, y0.clone(), slots)), tag
            _knobs(monkeypatch, MLORA_SLOT_KPARTS=None)
        else:
            assert torch.equal(got, _apply("mfma", proj, x, y0.clone(), slots)), tag


@pytest.mark.parametrize("rank,T,L", [(16, 256, 32), (8, 90, 12), (32, 200, 24), (64, 64, 7)])
def test_slot_major_grid_shares_long_k_out_between_the_workgroups_of_a_tile(rank, T, L, monkeypatch):
    """K = 4096: the four workgroups of a tile each multiply a quarter of K, publish their partial
    sums in the workspace, pick the others' up and expand a quarter of the columns.  Checked: the
    oracle's result; the same bits from one launch to the next, with the partners' words accepted,
    never accepted (every workgroup multiplies all parts itself) and not waited for; no wait running
    out in the ordinary runs; the workspace's generation one step on per launch with the arrival
    count back at zero; the same bits on a workspace that was never initialised; slot -1 rows untouched."""
    from nanovllm_voxcpm_amd import _hip, synthetic

    proj = _make("down", L, rank, torch.bfloat16, seed=180 + rank)
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=181, device="cuda")
    for tag, slots in _slot_form_batches(T, L, 182 + T).items():
        print(f"slot-major, K parts, r={rank} T={T} L={L} {tag}", flush=True)
        slots = slots.cuda()
        backend = _backend("slot")
        meta = _metadata(slots)

        def run():
            y = y0.clone()
            backend.add_lora([y], x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0)
            return y

        runs = []
        for spin in (20000, 20000, -1, 0):
            _knobs(monkeypatch, MLORA_SLOT_SPIN_TICKS=spin)
            runs.append(run())
            if spin > 0:
                assert _waits_run_out(backend) == 0, "a workgroup gave up waiting for its partners"
        exact, mag = _exact(proj, x, y0, slots)
        _check(runs[0], y0, exact, mag, slots, f"slot-major K parts/r{rank}/{tag}")
        for other in runs[1:]:
            assert torch.equal(runs[0], other), tag
        (scratch,) = backend._scratch.values()
        head = scratch[: _hip.WORKSPACE_HEAD_BYTES].view(torch.int32)
        want_check = ((len(runs) ^ 0x9E3779B9) + (1 << 31)) % (1 << 32) - (1 << 31)
        assert head[256 // 4 : 256 // 4 + 3].tolist() == [len(runs), 0, want_check]
        scratch[:4].zero_()  # no signature: nobody publishes, nobody waits
        _knobs(monkeypatch, MLORA_SLOT_SPIN_TICKS=20000)
        assert torch.equal(run(), runs[0])
        assert _waits_run_out(backend) == 0
        assert head[256 // 4 : 256 // 4 + 3].tolist() == [len(runs), 0, want_check]
    _knobs(monkeypatch, MLORA_SLOT_SPIN_TICKS=None)


@pytest.mark.parametrize("rank", [16, 64])
@pytest.mark.parametrize("name", ["gate_up", "o"])
def test_small_tile_form_is_the_same_for_every_column_range_width(name, rank, monkeypatch):
    """The small-tile kernel exists in an instance that requests one output span per wavefront up
    front (column ranges of at most 512 columns) and one that requests two (wider ranges); with
    ranges of 128..1024 columns both are taken, with and without the spans that wide ranges walk
    in a loop.  Every width gives the oracle's result, and all give the same bits: the cut into
    column ranges changes which workgroup computes a column, not how."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"small tiles, range widths, {name} r={rank}", flush=True)
    proj = _make(name, 32, rank, torch.bfloat16, seed=140 + rank)
    x, y0 = synthetic.make_activations(256, proj.k, sum(proj.widths), torch.bfloat16, seed=141, device="cuda")
    slots = synthetic.decode_slots(256, 32, seed=142).cuda()
    exact, mag = _exact(proj, x, y0, slots)
    outs = []
    for width in (128, 512, 1024, 4096):
        _knobs(monkeypatch, MLORA_DECODE_NT=width)
        outs.append(_apply("mfma", proj, x, y0.clone(), slots))
        _check(outs[-1], y0, exact, mag, slots, f"small tiles/{name}/r{rank}/ranges of {width}")
    _knobs(monkeypatch, MLORA_DECODE_NT=None)
    for out in outs[1:]:
        assert torch.equal(out, outs[0])


@pytest.mark.parametrize("sym", [0, 1])
@pytest.mark.parametrize("wide", [5, 7])
@pytest.mark.parametrize("kpart", [512, 1024])
@pytest.mark.parametrize("name,rank", [("down", 16), ("down", 64), ("qkv", 16), ("gate_up", 8), ("o", 32)])
def test_split_form_producers_and_consumers(name, rank, kpart, wide, sym, monkeypatch):
    """Small-tile form with the two products in different workgroups of one launch: producers
    publish the partial sums of their K part in the workspace, consumers pick them up (bounded
    wait) and expand their column range (sym: every workgroup is producer of a K part and consumer of
    a column range); a consumer whose wait runs out computes the sums itself.
    Checked: parity for both K-part widths, both role layouts and both access scopes, bit-identical results from one
    launch to the next and between accepting published sums, never accepting them and not waiting
    at all (the order of every sum is fixed, whatever the timing), slot -1 rows untouched, no wait
    running out in the ordinary runs, the arrival count back at zero and the generation one step on after each launch,
    and the same result from a workspace that was never initialised."""
    from nanovllm_voxcpm_amd import _hip, synthetic

    print(f"split form {name} r={rank} kpart={kpart} wide={wide} sym={sym}", flush=True)
    _knobs(monkeypatch, MLORA_SPLIT_KPART=kpart, MLORA_SPLIT_WIDE=wide, MLORA_SPLIT_SYM=sym, MLORA_SPLIT_W=128 if name == "qkv" else None)
    proj = _make(name, 12, rank, torch.bfloat16, seed=130 + rank)
    T = 90
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=131, device="cuda")
    g = torch.Generator().manual_seed(132)
    slots = torch.randint(-1, 12, (T,), generator=g, dtype=torch.int32)
    slots[:20] = 3  # one segment above the threshold: two small tiles of the same slot
    slots = slots.cuda()
    backend = _backend("split")
    meta = _metadata(slots)

    def run():
        y = y0.clone()
        blocks = list(y.split(proj.widths, dim=-1))
        backend.add_lora(blocks, x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0,
                         y_packed=y if len(blocks) > 1 else None)
        return y

    runs = []
    for spin in (20000, 20000, -1, 0):
        _knobs(monkeypatch, MLORA_SPLIT_SPIN_TICKS=spin)
        runs.append(run())
        if spin > 0:
            assert _waits_run_out(backend) == 0, "a consumer gave up waiting for its producers"
    exact, mag = _exact(proj, x, y0, slots)
    _check(runs[0], y0, exact, mag, slots, f"split/{name}/r{rank}/k{kpart}/w{wide}")
    for other in runs[1:]:
        assert torch.equal(runs[0], other)
    (scratch,) = backend._scratch.values()
    head = scratch[: _hip.WORKSPACE_HEAD_BYTES].view(torch.int32)
    state = head[256 // 4 : 256 // 4 + 2 * 1024].tolist()  # generation, arrivals, generation ^ check constant, then reserved words
    check = lambda gen: ((gen ^ 0x9E3779B9) + (1 << 31)) % (1 << 32) - (1 << 31)  # noqa: E731  (as the int32 word reads)
    assert state[:3] == [len(runs), 0, check(len(runs))] and not any(state[3:])  # one step per launch, arrivals back at zero
    # a head whose pair no longer fits its check word, or whose arrival count is impossible (memory that
    # was a workspace once and was handed out again in between can keep the signature): not believed,
    # not touched, same bits
    _knobs(monkeypatch, MLORA_SPLIT_SPIN_TICKS=20000)
    for gen, arrivals, chk in ((len(runs) + 5, 0, check(len(runs))), (len(runs), 1 << 20, check(len(runs)))):
        head[256 // 4 : 256 // 4 + 3] = torch.tensor([gen, arrivals, chk], dtype=torch.int32, device="cuda")
        assert torch.equal(run(), runs[0])
        assert head[256 // 4 : 256 // 4 + 3].tolist() == [gen, arrivals, chk]
    head[256 // 4 : 256 // 4 + 3] = torch.tensor(state[:3], dtype=torch.int32, device="cuda")
    # a workspace without the signature: same bits, nothing published, nobody waits
    scratch[:4].zero_()
    assert torch.equal(run(), runs[0])
    assert _waits_run_out(backend) == 0
    assert head[256 // 4 : 256 // 4 + 2 * 1024].tolist() == state


def test_split_form_ignores_what_a_launch_of_another_layout_left():
    """Two projections of different shape share one workspace, as the layers of a model do.  The
    first launch (three slices, few tiles) leaves tagged sums all over the exchange area; the second
    (one slice, long K, more tiles, among them tiles the first never had) lays its own sums out
    differently over the same bytes.  Its consumers must not take any of the old words for new ones:
    same bits as on a workspace nobody used before, in either order of the two launches."""
    from nanovllm_voxcpm_amd import synthetic

    shapes = {"three": (1024, [512, 128, 128]), "long": (4096, [1024])}
    projs = {n: synthetic.make_projection(n, 24, 32, torch.bfloat16, seed=150, device="cuda", shapes=shapes) for n in shapes}
    g = torch.Generator().manual_seed(151)
    few = torch.randint(0, 3, (40,), generator=g, dtype=torch.int32).cuda()      # three slots: three or four tiles
    many = torch.randint(-1, 24, (200,), generator=g, dtype=torch.int32).cuda()  # every slot: thirty tiles or so
    batches = {"three": few, "long": many}
    data = {n: synthetic.make_activations(batches[n].numel(), projs[n].k, sum(projs[n].widths), torch.bfloat16, seed=152, device="cuda") for n in shapes}

    def run(backend, n):
        x, y0 = data[n]
        y = y0.clone()
        blocks = list(y.split(projs[n].widths, dim=-1))
        backend.add_lora(blocks, x, projs[n].a, projs[n].b, indices=batches[n], metadata=_metadata(batches[n]), scaling=1.0,
                         y_packed=y if len(blocks) > 1 else None)
        return y

    fresh = {n: run(_backend("split"), n) for n in shapes}
    for order in (("three", "long"), ("long", "three"), ("three", "three", "long", "long", "three")):
        shared = _backend("split")
        for n in order:
            assert torch.equal(run(shared, n), fresh[n]), f"{n} after {order}"
        assert _waits_run_out(shared) == 0
    for n in shapes:
        x, y0 = data[n]
        exact, mag = _exact(projs[n], x, y0, batches[n])
        _check(fresh[n], y0, exact, mag, batches[n], f"split/shared-workspace/{n}")


def test_config2_matches_reference_torch_loop():
    """The same batch against the reference's torch formulation (per-token F.linear loop) on the
    host.  With fp32 accumulation (the loop run on fp32 copies of the bf16 values) every element
    meets the stated tolerance.  Run in bf16 end to end, that loop rounds the intermediate, the
    update and the sum separately, which alone can leave it two output ulps (1.6 %) from the
    exact value, so against it only the bulk of the elements is held to the tolerance."""
    from nanovllm_voxcpm_amd import synthetic

    proj = _make("qkv", 32, 16, torch.bfloat16, seed=100)
    x, y0 = synthetic.make_activations(256, proj.k, sum(proj.widths), torch.bfloat16, seed=101, device="cuda")
    slots = synthetic.decode_slots(256, 32, seed=102)
    got = _apply("auto", proj, x, y0.clone(), slots.cuda()).cpu().float()
    a_cpu, b_cpu = [a.cpu() for a in proj.a], [b.cpu() for b in proj.b]
    y32 = y0.cpu().float()
    oracle.per_token_add_lora(list(y32.split(proj.widths, dim=-1)), x.cpu().float(), [a.float() for a in a_cpu],
                              [b.float() for b in b_cpu], indices=slots, scaling=1.0, y_packed=y32)
    assert torch.allclose(got, y32, rtol=RTOL, atol=ATOL)
    y16 = y0.cpu().clone()
    oracle.per_token_add_lora(list(y16.split(proj.widths, dim=-1)), x.cpu(), a_cpu, b_cpu, indices=slots, scaling=1.0, y_packed=y16)
    close = torch.isclose(got, y16.float(), rtol=RTOL, atol=ATOL)
    assert close.float().mean().item() > 0.999
    assert (got - y16.float()).abs().max().item() < 2.0 ** -5  # two ulps of the largest outputs


@pytest.mark.parametrize("form", ["bgmv", "mfma", "token"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rank", [8, 16, 32, 64])
def test_ranks_and_dtypes_small(rank, dtype, form):
    from nanovllm_voxcpm_amd import synthetic

    print(f"ranks rank={rank} dtype={dtype} form={form}", flush=True)
    shapes = {"p": (256, [64, 136, 8])}  # widths that are not multiples of the column tiles
    proj = synthetic.make_projection("p", 6, rank, dtype, seed=7 + rank, device="cuda", shapes=shapes)
    x, y0 = synthetic.make_activations(75, 256, 208, dtype, seed=9, device="cuda")
    g = torch.Generator().manual_seed(rank)
    slots = torch.randint(-1, 6, (75,), generator=g, dtype=torch.int32).cuda()
    got = _apply(form, proj, x, y0.clone(), slots, scaling=0.5)
    exact, mag = _exact(proj, x, y0, slots, scaling=0.5)
    _check(got, y0, exact, mag, slots, f"rank{rank}/{dtype}/{form}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rank", [24, 40, 48, 56])
def test_ranks_between_the_kernel_instances_run_on_the_matrix_cores(rank, dtype):
    """Buffers of rank 24, 40, 48, 56 (the reference takes any max_lora_rank): the small-tile kernels
    of the next rank up take them with the buffers' rank as stride and everything beyond it masked.
    Ragged widths at K = 256 (the general instance), the four projection shapes at decode size (staged
    instance, slot-major grid, K shared out at 4096) and a 1500-token batch; NaN beyond every slot's
    own rank; a slot vector with rows without adapter.  AUTO and the forms it picks from give the
    fp64 result; the forms that take exact ranks only say so."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"in-between rank {rank} {dtype}", flush=True)
    shapes = {"p": (256, [64, 136, 8])}
    proj = synthetic.make_projection("p", 6, rank, dtype, seed=17 + rank, device="cuda", shapes=shapes)
    x, y0 = synthetic.make_activations(75, 256, 208, dtype, seed=19, device="cuda")
    g = torch.Generator().manual_seed(rank)
    slots = torch.randint(-1, 6, (75,), generator=g, dtype=torch.int32).cuda()
    exact, mag = _exact(proj, x, y0, slots, scaling=0.5)
    for form in ("auto", "mfma", "token"):
        _check(_apply(form, proj, x, y0.clone(), slots, scaling=0.5), y0, exact, mag, slots, f"rank{rank}/{dtype}/{form}")
    for form in ("sgmv", "split", "bgmv"):
        with pytest.raises(RuntimeError, match="rank"):
            _apply(form, proj, x, y0.clone(), slots)
    for name, T in (("qkv", 256), ("o", 256), ("gate_up", 256), ("down", 256), ("o", 1500)):
        true_ranks = [rank, 8, rank - 8, rank, 16, 0, rank, rank - 4]
        clean = _make(name, len(true_ranks), rank, dtype, seed=27 + rank, true_ranks=true_ranks)
        a_nan, b_nan = [t.clone() for t in clean.a], [t.clone() for t in clean.b]
        for sl, r in enumerate(true_ranks):
            for t in a_nan:
                t[sl, r:] = float("nan")
            for t in b_nan:
                t[sl, :, r:] = float("nan")
        x, y0 = synthetic.make_activations(T, clean.k, sum(clean.widths), dtype, seed=29, device="cuda")
        slots = torch.randint(-1, len(true_ranks), (T,), generator=g, dtype=torch.int32).cuda()
        exact, mag = _exact(clean, x, y0, slots)
        eff = torch.tensor(true_ranks, dtype=torch.int32, device="cuda")
        forms = ["auto", "mfma"] + (["slot"] if name != "qkv" else [])
        for form in forms:
            # without the rank vector (zero padding inside the buffers' rank) and with it (NaN there)
            _check(_apply(form, clean, x, y0.clone(), slots), y0, exact, mag, slots, f"rank{rank}/{name}/T{T}/{form}")
            y = y0.clone()
            blocks = list(y.split(clean.widths, dim=-1))
            _backend(form).add_lora(blocks, x, a_nan, b_nan, indices=slots, metadata=_metadata(slots), scaling=1.0,
                                    y_packed=y if len(blocks) > 1 else None, effective_rank=eff)
            assert torch.isfinite(y.float()).all()
            _check(y, y0, exact, mag, slots, f"rank{rank}/{name}/T{T}/{form}/masked")


@pytest.mark.parametrize("rank", [1, 3, 4, 12, 72, 128])
def test_ranks_the_vector_kernels_do_not_take_go_through_the_token_kernel(rank):
    """Ranks that are not a multiple of eight (rows of B then do not start on 16-byte boundaries) or
    lie above 64: AUTO takes the one-workgroup-per-token kernel, with the oracle's result."""
    from nanovllm_voxcpm_amd import synthetic

    shapes = {"p": (256, [64, 136, 8])}
    proj = synthetic.make_projection("p", 5, rank, torch.bfloat16, seed=37 + rank, device="cuda", shapes=shapes)
    x, y0 = synthetic.make_activations(60, 256, 208, torch.bfloat16, seed=39, device="cuda")
    g = torch.Generator().manual_seed(rank)
    slots = torch.randint(-1, 5, (60,), generator=g, dtype=torch.int32).cuda()
    exact, mag = _exact(proj, x, y0, slots)
    _check(_apply("auto", proj, x, y0.clone(), slots), y0, exact, mag, slots, f"rank{rank}/auto")


@pytest.mark.parametrize("staged", ["1", "0"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rank", [8, 16, 32, 64])
def test_small_tile_form_shapes(rank, dtype, staged, monkeypatch):
    """The small-tile kernel at the K values that select its specialisations (1024, 2048, 3072:
    4096: four, eight, twelve, sixteen k-steps per wavefront with staged operands; 512 and 160: two
    k-steps / run-time split),
    with ragged slice widths, narrow and wide column ranges,
    row-strided x and y views, rows without adapter and a segment longer than one tile."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"small tiles r={rank} {dtype} staged={staged}", flush=True)
    _knobs(monkeypatch, MLORA_DECODE_STAGED=staged)
    shapes = {"a": (1024, [72, 200, 8]), "b": (4096, [328]), "c": (512, [1096, 64]), "d": (160, [24]),
              "e": (2048, [136, 64]), "f": (3072, [72])}  # 8, 12 and (K = 4096) 16 k-steps per wavefront
    g = torch.Generator().manual_seed(40 + rank)
    T = 77
    slots = torch.randint(-1, 9, (T,), generator=g, dtype=torch.int32)
    slots[5:30] = 4
    slots = slots.cuda()
    for name in shapes:
        proj = synthetic.make_projection(name, 9, rank, dtype, seed=950 + rank, device="cuda", shapes=shapes)
        xw, yw = synthetic.make_activations(T, proj.k + 16, sum(proj.widths) + 24, dtype, seed=951, device="cuda")
        x, y0 = xw[:, 8 : 8 + proj.k], yw[:, 8 : 8 + sum(proj.widths)]
        y = yw.clone()[:, 8 : 8 + sum(proj.widths)]
        got = _apply("mfma", proj, x, y, slots, scaling=1.25)
        exact, mag = _exact(proj, x, y0, slots, scaling=1.25)
        _check(got, y0, exact, mag, slots, f"small/{name}/r{rank}/{dtype}/staged{staged}")
        assert torch.equal(y._base[:, :8], yw[:, :8]) and torch.equal(y._base[:, 8 + sum(proj.widths):], yw[:, 8 + sum(proj.widths):])


@pytest.mark.parametrize("form", ["auto", "token"])
def test_odd_shapes_take_the_scalar_path(form):
    """K, widths and rank that are not multiples of eight, unaligned column offsets, fp32."""
    g = torch.Generator().manual_seed(21)
    for dtype in (torch.float32, torch.bfloat16):
        T, K, r, L = 19, 37, 5, 3
        widths = [11, 3]
        x = torch.randn(T, K, generator=g).to(dtype).cuda()
        y0 = torch.randn(T, sum(widths), generator=g).to(dtype).cuda()
        a = [(torch.randn(L, r, K, generator=g) * 0.3).to(dtype).cuda() for _ in widths]
        b = [(torch.randn(L, n, r, generator=g) * 0.3).to(dtype).cuda() for n in widths]
        slots = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32).cuda()
        y = y0.clone()
        _backend(form).add_lora(list(y.split(widths, dim=-1)), x, a, b, indices=slots, metadata=_metadata(slots), scaling=1.5, y_packed=y)
        want = oracle.fused_add_lora(list(y0.cpu().split(widths, dim=-1)), x.cpu(), [t.cpu() for t in a], [t.cpu() for t in b],
                                     indices=slots.cpu(), scaling=1.5, accumulate=torch.float64)
        tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=RTOL, atol=ATOL)
        assert torch.allclose(y.cpu().double(), torch.cat(want, dim=-1).double(), **tol)


# ---- config 3: prefill, 16 sequences, 8 adapters of rank 64, a quarter without adapter ------------


@pytest.mark.parametrize("form", ["auto", "sgmv", "wide", "mfma", "bgmv"])
@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
def test_config3_prefill_bf16(name, form):
    from nanovllm_voxcpm_amd import synthetic

    print(f"config3 {name} form={form}", flush=True)
    proj = _make(name, 8, 64, torch.bfloat16, seed=300)
    if name in ("gate_up", "down") or form == "bgmv":
        # same mix of sequences, shorter ones: bounds the host-side fp64 check
        slots_cpu, lengths = synthetic.prefill_slots(16, 8, seed=301, min_len=16, max_len=160)
    else:
        slots_cpu, lengths = synthetic.prefill_slots(16, 8, seed=301)
    T = slots_cpu.numel()
    assert (slots_cpu < 0).any() and (slots_cpu >= 0).any()
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=302, device="cuda")
    slots = slots_cpu.cuda()
    got = _apply(form, proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, f"config3/{name}/{form}")


@pytest.mark.parametrize("knobs", [{}, {"MLORA_SGMV_KSPLIT": "1", "MLORA_SGMV_GROUP": "2"}, {"MLORA_SGMV_KR": "128", "MLORA_SGMV_KSPLIT": "4", "MLORA_SGMV_GROUP": "4", "MLORA_SGMV_CPL": "4"},
                                   {"MLORA_SGMV_ALL_SLICES": "2", "MLORA_SGMV_KR": "256", "MLORA_SGMV_NT": "512"},
                                   {"MLORA_SGMV_XDB": "0", "MLORA_SGMV_KSPLIT": "1"}])  # K parts of several one-slab batches
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rank", [8, 16, 32, 64])
def test_long_segment_form_shapes(rank, dtype, knobs, monkeypatch):
    """The two-launch form on segments of 1..130 tokens (short ones, exact tile multiples, tails),
    rows without adapter, ragged slice widths (not multiples of a span), row-strided x and y
    views, every rank and both 16-bit types, and the launch shapes the knobs select (K parts,
    slab width, tile groups, span width, slice walk)."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"long form r={rank} {dtype} {knobs}", flush=True)
    for key, value in knobs.items():
        monkeypatch.setenv(key, value)
    _knobs(monkeypatch)
    # K = 640 and 768 take 128- and 256-column x batches, 1536 and 2048 several batches per K part
    shapes = {"p": (512, [72, 200, 8]), "q": (1024, [520]), "s": (640, [64, 72]), "t": (768, [264]), "u": (1536, [136]), "v": (2048, [64])}
    lengths = [130, 1, 64, 15, 16, 65, 3, 128, 17, 7]
    slot_of = [2, 0, 5, 1, 3, -1, 4, 2, -1, 6]  # slot 2 twice: two segments merge into one of 258
    slots = torch.cat([torch.full((n,), s, dtype=torch.int32) for n, s in zip(lengths, slot_of)])
    slots = slots[torch.randperm(slots.numel(), generator=torch.Generator().manual_seed(9))].cuda()
    T = slots.numel()
    for name in shapes:
        proj = synthetic.make_projection(name, 7, rank, dtype, seed=900 + rank, device="cuda", shapes=shapes)
        xw, yw = synthetic.make_activations(T, proj.k + 24, sum(proj.widths) + 40, dtype, seed=901, device="cuda")
        x, y0 = xw[:, 8 : 8 + proj.k], yw[:, 16 : 16 + sum(proj.widths)]  # 16-byte aligned views of wider buffers
        y = yw.clone()[:, 16 : 16 + sum(proj.widths)]
        got = _apply("sgmv", proj, x, y, slots, scaling=0.75)
        exact, mag = _exact(proj, x, y0, slots, scaling=0.75)
        _check(got, y0, exact, mag, slots, f"long/{name}/r{rank}/{dtype}/{knobs}")
        assert torch.equal(y._base[:, :16], yw[:, :16]) and torch.equal(y._base[:, 16 + sum(proj.widths):], yw[:, 16 + sum(proj.widths):])


@pytest.mark.parametrize("nt", [0, 512, 2048])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rank", [8, 16, 32, 64])
def test_one_launch_form_over_64_token_tiles_shapes(rank, dtype, nt, monkeypatch):
    """The one-launch form whose workgroups shrink their tile themselves, on the shapes of the
    two-launch form's test: segments of 1..130 tokens (short ones, exact tile multiples, tails),
    rows without adapter, ragged slice widths, row-strided x and y views, K of 128- and 256-column
    batches and of many batches, every rank, both 16-bit types, narrow and wide column ranges."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"one-launch form over 64-token tiles r={rank} {dtype} nt={nt}", flush=True)
    _knobs(monkeypatch, MLORA_WIDE_NT=nt or None)
    shapes = {"p": (512, [72, 200, 8]), "q": (1024, [520]), "s": (640, [64, 72]), "t": (768, [264]), "u": (1536, [136]), "v": (2048, [64]),
              "w": (256, [2600, 1032])}
    lengths = [130, 1, 64, 15, 16, 65, 3, 128, 17, 7]
    slot_of = [2, 0, 5, 1, 3, -1, 4, 2, -1, 6]  # slot 2 twice: two segments merge into one of 258
    slots = torch.cat([torch.full((n,), s, dtype=torch.int32) for n, s in zip(lengths, slot_of)])
    slots = slots[torch.randperm(slots.numel(), generator=torch.Generator().manual_seed(9))].cuda()
    T = slots.numel()
    for name in shapes:
        proj = synthetic.make_projection(name, 7, rank, dtype, seed=900 + rank, device="cuda", shapes=shapes)
        xw, yw = synthetic.make_activations(T, proj.k + 24, sum(proj.widths) + 40, dtype, seed=901, device="cuda")
        x, y0 = xw[:, 8 : 8 + proj.k], yw[:, 16 : 16 + sum(proj.widths)]  # 16-byte aligned views of wider buffers
        y = yw.clone()[:, 16 : 16 + sum(proj.widths)]
        got = _apply("wide", proj, x, y, slots, scaling=0.75)
        exact, mag = _exact(proj, x, y0, slots, scaling=0.75)
        _check(got, y0, exact, mag, slots, f"wide/{name}/r{rank}/{dtype}/nt{nt}")
        assert torch.equal(y._base[:, :16], yw[:, :16]) and torch.equal(y._base[:, 16 + sum(proj.widths):], yw[:, 16 + sum(proj.widths):])
        assert torch.equal(got, _apply("wide", proj, x, yw.clone()[:, 16 : 16 + sum(proj.widths)], slots, scaling=0.75))  # the same bits again
    _knobs(monkeypatch, MLORA_WIDE_NT=None)


def test_workgroups_of_one_blockidx_x_share_an_xcd():
    """Grids of x extent 8: the kernels treat blockIdx.x as the XCD (column ranges of a tile share
    an L2; workgroups that hand each other partial sums through it check the XCD they ran on).
    Every workgroup records its XCD: one XCD per blockIdx.x, whatever y and z."""
    from nanovllm_voxcpm_amd import _hip

    grid = (8, 5, 37)
    out = torch.full((grid[0] * grid[1] * grid[2],), -1, dtype=torch.int32, device="cuda")
    _hip.probe_launch(3, out, grid=grid, threads=256)
    torch.cuda.synchronize()
    xcd = out.cpu().view(grid[2], grid[1], grid[0])
    assert (xcd >= 0).all()
    for bx in range(8):
        assert xcd[:, :, bx].unique().numel() == 1, f"blockIdx.x = {bx} ran on XCDs {xcd[:, :, bx].unique().tolist()}"
    print("XCD of blockIdx.x 0..7:", [int(xcd[0, 0, bx]) for bx in range(8)], flush=True)


@pytest.mark.parametrize("knobs", [{}, {"MLORA_SGMV_KSPLIT": "1", "MLORA_SGMV_GROUP": "4"}, {"MLORA_SGMV_KSPLIT": "4", "MLORA_SGMV_GROUP": "1", "MLORA_SGMV_NT": "512"},
                                   {"MLORA_SGMV_ALL_SLICES": "2", "MLORA_SGMV_GROUP": "4", "MLORA_SGMV_NT": "512"}])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rank", [8, 16, 32, 64])
def test_long_segment_form_in_one_launch(rank, dtype, knobs, monkeypatch):
    """The one-launch form of the long-segment kernels: the workgroups of a group of tiles share
    out its shrink, seal what they wrote, wait for each other's seals (bounded) and expand a column
    range each.  Same batch as for the two-launch form (segments of 1..130 tokens, rows without
    adapter, ragged widths, strided views).  Checked: parity; the bits of the two-launch form where
    neither cuts K (same sums, same order); the same bits on a second launch, when no seal is ever accepted
    (every workgroup computes what it needs itself) and on a workspace without the signature; no
    wait running out in the ordinary runs; the arrival count back at zero and the generation one
    step on after each launch."""
    from nanovllm_voxcpm_amd import _hip, synthetic

    print(f"one-launch long form r={rank} {dtype} {knobs}", flush=True)
    for key, value in knobs.items():
        monkeypatch.setenv(key, value)
    _knobs(monkeypatch)
    shapes = {"p": (512, [72, 200, 8]), "q": (1024, [520]), "t": (768, [264]), "u": (1536, [136]), "v": (2048, [64])}
    lengths = [130, 1, 64, 15, 16, 65, 3, 128, 17, 7]
    slot_of = [2, 0, 5, 1, 3, -1, 4, 2, -1, 6]  # slot 2 twice: two segments merge into one of 258
    slots = torch.cat([torch.full((n,), s, dtype=torch.int32) for n, s in zip(lengths, slot_of)])
    slots = slots[torch.randperm(slots.numel(), generator=torch.Generator().manual_seed(9))].cuda()
    T = slots.numel()
    for name in shapes:
        proj = synthetic.make_projection(name, 7, rank, dtype, seed=900 + rank, device="cuda", shapes=shapes)
        xw, yw = synthetic.make_activations(T, proj.k + 24, sum(proj.widths) + 40, dtype, seed=901, device="cuda")
        x, y0 = xw[:, 8 : 8 + proj.k], yw[:, 16 : 16 + sum(proj.widths)]  # 16-byte aligned views of wider buffers
        backend = _backend("fused")
        meta = _metadata(slots)

        def run():
            y = yw.clone()[:, 16 : 16 + sum(proj.widths)]
            blocks = list(y.split(proj.widths, dim=-1))
            backend.add_lora(blocks, x, proj.a, proj.b, indices=slots, metadata=meta, scaling=0.75, y_packed=y if len(blocks) > 1 else None)
            return y

        runs = []
        for spin in (50000, 50000, -1):
            _knobs(monkeypatch, MLORA_FUSED_SPIN_TICKS=spin)
            runs.append(run())
            if spin > 0:
                assert _waits_run_out(backend) == 0, "a workgroup gave up waiting for its unit's seals"
        got = runs[0]
        exact, mag = _exact(proj, x, y0, slots, scaling=0.75)
        _check(got, y0, exact, mag, slots, f"one-launch/{name}/r{rank}/{dtype}/{knobs}")
        assert torch.equal(got._base[:, :16], yw[:, :16]) and torch.equal(got._base[:, 16 + sum(proj.widths):], yw[:, 16 + sum(proj.widths):])
        for other in runs[1:]:
            assert torch.equal(got, other)
        two = _apply("sgmv", proj, x, yw.clone()[:, 16 : 16 + sum(proj.widths)], slots, scaling=0.75)
        if knobs.get("MLORA_SGMV_KSPLIT") == "1":  # K uncut in both forms: the same sums in the same order
            assert torch.equal(got, two)
        else:
            assert torch.allclose(got.float(), two.float(), rtol=RTOL, atol=ATOL)
        (scratch,) = backend._scratch.values()
        head = scratch[: _hip.WORKSPACE_HEAD_BYTES].view(torch.int32)
        state = head[256 // 4 : 256 // 4 + 2 * 1024].tolist()  # generation, arrivals, generation ^ check constant, then reserved words
        want_check = ((len(runs) ^ 0x9E3779B9) + (1 << 31)) % (1 << 32) - (1 << 31)
        assert state[:3] == [len(runs), 0, want_check] and not any(state[3:])  # one step per launch, arrivals back at zero
        # a workspace without the signature: nobody seals, nobody waits, same bits
        scratch[:4].zero_()
        _knobs(monkeypatch, MLORA_FUSED_SPIN_TICKS=50000)
        assert torch.equal(run(), got)
        assert _waits_run_out(backend) == 0
        assert head[256 // 4 : 256 // 4 + 2 * 1024].tolist() == state


@pytest.mark.parametrize("name,rank,expected", [("o", 16, "mfma"), ("o", 64, "wide"), ("gate_up", 64, "sgmv"), ("down", 64, "sgmv")])
def test_auto_form_follows_rank_and_width(name, rank, expected):
    """A 3000-token prefill of three sequences: at rank 16 the one-launch small-tile form is the
    faster one up to far larger batches; at rank 64 the forms over 64-token tiles take over near
    8500 tokens (here 12000): the one-launch form where a tile's column ranges repeat little of its
    shrink (o), the two-launch form elsewhere (gate_up: many ranges, down: a long K).  AUTO gives
    the oracle's result in every case and exactly what the form it is meant to pick gives."""
    print(f"auto form {name} r={rank}", flush=True)
    T = 3000 if rank == 16 else 12000
    proj = _make(name, 4, rank, torch.bfloat16, seed=330 + rank)
    slots = torch.cat([torch.full((T // 2,), 1, dtype=torch.int32), torch.full((T // 4,), -1, dtype=torch.int32),
                       torch.full((T - T // 2 - T // 4,), 3, dtype=torch.int32)]).cuda()
    from nanovllm_voxcpm_amd import synthetic

    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=331, device="cuda")
    got = _apply("auto", proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, f"auto/{name}/r{rank}")
    assert torch.equal(got, _apply(expected, proj, x, y0.clone(), slots))


@pytest.mark.parametrize("rank", [16, 32, 64])
def test_auto_shares_k_of_4096_out_in_the_slot_major_form(rank):
    """down of the decode batch: AUTO takes the slot-major form, whose workgroups share K out between
    them, at every rank (where the split form used to be taken for ranks 32 and 64)."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"auto, K = 4096, r={rank}", flush=True)
    proj = _make("down", 32, rank, torch.bfloat16, seed=345 + rank)
    x, y0 = synthetic.make_activations(256, proj.k, sum(proj.widths), torch.bfloat16, seed=346, device="cuda")
    slots = synthetic.decode_slots(256, 32, seed=347).cuda()
    got = _apply("auto", proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, f"auto/down/r{rank}")
    assert torch.equal(got, _apply("slot", proj, x, y0.clone(), slots))


@pytest.mark.parametrize("rank", [16, 32])
def test_auto_takes_the_split_form_for_very_long_k(rank):
    """K = 8192 (a model eight times as wide): a workgroup's K range no longer fits its registers as
    one batch of loads, so AUTO lets the workgroups of a tile share the shrink.  Parity, and the
    same bits as the form it is meant to pick."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"auto split r={rank}", flush=True)
    shapes = {"wide_down": (8192, [1024, 264])}
    proj = synthetic.make_projection("wide_down", 6, rank, torch.bfloat16, seed=340 + rank, device="cuda", shapes=shapes)
    x, y0 = synthetic.make_activations(70, proj.k, sum(proj.widths), torch.bfloat16, seed=341, device="cuda")
    g = torch.Generator().manual_seed(342)
    slots = torch.randint(-1, 6, (70,), generator=g, dtype=torch.int32).cuda()
    got = _apply("auto", proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, f"auto-split/r{rank}")
    assert torch.equal(got, _apply("split", proj, x, y0.clone(), slots))
    assert torch.allclose(got.float(), _apply("mfma", proj, x, y0.clone(), slots).float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed", list(range(32)))
def test_seeded_random_shapes_all_forms_agree_with_the_oracle(seed):
    """Shapes nobody picked by hand: token counts 1..2500, 1..40 slots, K a multiple of 32 (so
    also of 64 and 128 in some draws, which decides which kernels may run), one to three slices
    of ragged widths, a random share of rows without adapter, random segment structure (sorted
    runs or fully shuffled), views of wider buffers.  Every form that accepts the shape gives the
    oracle's result."""
    g = torch.Generator().manual_seed(7000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    rank = (8, 16, 32, 64)[ri(0, 3)]
    dtype = (torch.bfloat16, torch.float16)[ri(0, 1)]
    T, L = (1, 7, 40, 300, 1100, 2500)[ri(0, 5)], (1, 3, 9, 40)[ri(0, 3)]
    K = 32 * ri(1, 40) if ri(0, 1) else 128 * ri(1, 16)
    widths = [8 * ri(1, 96) for _ in range(ri(1, 3))]
    print(f"random seed={seed} r={rank} {dtype} T={T} L={L} K={K} widths={widths}", flush=True)
    slots = torch.randint(0, L, (T,), generator=g, dtype=torch.int32)
    if ri(0, 1):
        slots = torch.sort(slots).values  # long runs, as a prefill batch has them
    slots[torch.rand(T, generator=g) < (0.0, 0.2, 0.7)[ri(0, 2)]] = -1
    slots = slots.cuda()
    a = [(torch.randn(L, rank, K, generator=g) * 0.05).to(dtype).cuda() for _ in widths]
    b = [(torch.randn(L, n, rank, generator=g) * 0.05).to(dtype).cuda() for n in widths]
    from nanovllm_voxcpm_amd import synthetic

    proj = synthetic.ProjectionWeights("random", K, widths, a, b)
    pad_x, pad_y = 8 * ri(0, 2), 8 * ri(0, 2)
    xw = torch.randn(T, K + 2 * pad_x, generator=g).to(dtype).cuda()
    yw = torch.randn(T, sum(widths) + 2 * pad_y, generator=g).to(dtype).cuda()
    x, y0 = xw[:, pad_x : pad_x + K], yw[:, pad_y : pad_y + sum(widths)]
    exact, mag = _exact(proj, x, y0, slots, scaling=0.5)
    forms = ["auto", "token", "bgmv", "mfma"] + (["sgmv", "wide"] if K % 128 == 0 else [])
    for form in forms:
        y = yw.clone()[:, pad_y : pad_y + sum(widths)]
        got = _apply(form, proj, x, y, slots, scaling=0.5)
        _check(got, y0, exact, mag, slots, f"random/{seed}/{form}")
        assert torch.equal(y._base[:, :pad_y], yw[:, :pad_y]) and torch.equal(y._base[:, pad_y + sum(widths):], yw[:, pad_y + sum(widths):])


# ---- config 4: mixed batch, 128 adapters of ranks {8,16,32,64} padded to 64, Zipf popularity ----


@pytest.mark.parametrize("name", ["qkv", "down"])
def test_config4_mixed_batch_rank_masking(name):
    from nanovllm_voxcpm_amd import synthetic

    print(f"config4 {name}", flush=True)
    ranks = synthetic.heterogeneous_ranks(128, seed=400)
    proj = _make(name, 128, 64, torch.bfloat16, seed=401, true_ranks=ranks)
    slots_cpu = synthetic.mixed_slots(seed=402)
    assert slots_cpu.numel() == 8192
    x, y0 = synthetic.make_activations(8192, proj.k, sum(proj.widths), torch.bfloat16, seed=403, device="cuda")
    slots = slots_cpu.cuda()
    got = _apply("auto", proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, f"config4/{name}")
    # rank padding is inert: the same adapters stored at their true rank in rank-r buffers of a
    # narrower layer give the same result for the slots whose rank fits
    narrow = [s for s, r in enumerate(ranks) if r <= 16]
    keep = torch.tensor([s in set(narrow) for s in slots_cpu.tolist()])
    slots16 = torch.where(keep, slots_cpu, torch.full_like(slots_cpu, -1)).cuda()
    proj16 = synthetic.ProjectionWeights(proj.name, proj.k, proj.widths, [a[:, :16].contiguous() for a in proj.a], [b[:, :, :16].contiguous() for b in proj.b])
    got16 = _apply("auto", proj16, x, y0.clone(), slots16)
    got64 = _apply("auto", proj, x, y0.clone(), slots16)
    assert torch.allclose(got16.float(), got64.float(), rtol=RTOL, atol=ATOL)


# ---- size-independent properties at full size ----------------------------------------------------


def test_full_size_properties_gate_up_prefill():
    from nanovllm_voxcpm_amd import synthetic

    proj = _make("gate_up", 8, 64, torch.bfloat16, seed=500)
    slots_cpu, _ = synthetic.prefill_slots(16, 8, seed=501)
    T = slots_cpu.numel()
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=502, device="cuda")
    slots = slots_cpu.cuda()
    got = _apply("auto", proj, x, y0.clone(), slots)
    live = slots >= 0
    assert torch.equal(got[~live], y0[~live])                      # pass-through
    assert not torch.equal(got[live], y0[live])
    zero_a = synthetic.ProjectionWeights(proj.name, proj.k, proj.widths, [torch.zeros_like(a) for a in proj.a], proj.b)
    assert torch.equal(_apply("auto", zero_a, x, y0.clone(), slots), y0)   # zero A => y unchanged
    # linearity in B on a zero base: doubling B doubles the update exactly (powers of two)
    z = torch.zeros_like(y0)
    d1 = _apply("auto", proj, x, z.clone(), slots)
    twice = synthetic.ProjectionWeights(proj.name, proj.k, proj.widths, proj.a, [b * 2 for b in proj.b])
    d2 = _apply("auto", twice, x, z.clone(), slots)
    assert torch.equal(d2, d1 * 2)
    # permuting the tokens permutes the result
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(5)).cuda()
    got_p = _apply("auto", proj, x[perm].contiguous(), y0[perm].contiguous(), slots[perm].contiguous())
    assert torch.allclose(got_p.float(), got[perm].float(), rtol=RTOL, atol=ATOL)
    # kernel families agree with each other
    got_b = _apply("bgmv", proj, x, y0.clone(), slots)
    assert torch.allclose(got_b.float(), got.float(), rtol=RTOL, atol=ATOL)


def test_empty_and_degenerate_batches():
    from nanovllm_voxcpm_amd import synthetic
    from nanovllm_voxcpm_amd.lora import LoRAMetadata

    proj = _make("o", 4, 16, torch.bfloat16, seed=600)
    backend = _backend()
    # all rows without adapter
    x, y0 = synthetic.make_activations(33, 1024, 1024, torch.bfloat16, seed=601, device="cuda")
    slots = torch.full((33,), -1, dtype=torch.int32, device="cuda")
    assert torch.equal(_apply("auto", proj, x, y0.clone(), slots), y0)
    assert torch.equal(_apply("token", proj, x, y0.clone(), slots), y0)
    # no_lora_flag short-circuits without reading anything
    meta = LoRAMetadata(slots, None, None, None, None, True, 0)
    y = y0.clone()
    backend.add_lora([y], x, proj.a, proj.b, indices=slots, metadata=meta, scaling=1.0)
    assert torch.equal(y, y0)
    # zero tokens
    xe, ye = x[:0], y0[:0].clone()
    se = slots[:0]
    assert backend.add_lora([ye], xe, proj.a, proj.b, indices=se, metadata=_metadata(se), scaling=1.0)[0].shape == (0, 1024)
    assert backend.add_lora([], x, [], [], indices=slots, metadata=_metadata(slots), scaling=1.0) == []
    # one token, one slot; every token on one slot (a single long segment)
    for T in (1, 700):
        x, y0 = synthetic.make_activations(T, 1024, 1024, torch.bfloat16, seed=602, device="cuda")
        slots = torch.full((T,), 3, dtype=torch.int32, device="cuda")
        got = _apply("auto", proj, x, y0.clone(), slots)
        exact, mag = _exact(proj, x, y0, slots)
        _check(got, y0, exact, mag, slots, f"single-slot T={T}")
    # a slot id beyond the resident slots is treated as "no adapter"
    slots = torch.tensor([0, 9, 1], dtype=torch.int32, device="cuda")
    x, y0 = synthetic.make_activations(3, 1024, 1024, torch.bfloat16, seed=603, device="cuda")
    got = _apply("auto", proj, x, y0.clone(), slots)
    assert torch.equal(got[1], y0[1]) and not torch.equal(got[0], y0[0])


def test_strided_views_and_3d_inputs():
    """x / y that are column blocks of wider buffers (row stride > width) and a 3-D batch through a layer."""
    from nanovllm_voxcpm_amd import synthetic
    from nanovllm_voxcpm_amd.layers.lora import LoRALinear
    from nanovllm_voxcpm_amd.utils.context import build_lora_context_from_token_to_slot, set_lora_context

    proj = _make("o", 4, 16, torch.bfloat16, seed=700)
    xw, yw = synthetic.make_activations(40, 2048, 3072, torch.bfloat16, seed=701, device="cuda")
    x, y = xw[:, 512:1536], yw[:, 1024:2048]
    y0 = yw.clone()
    slots = synthetic.decode_slots(40, 4, seed=702).cuda()
    _backend().add_lora([y], x, proj.a, proj.b, indices=slots, metadata=_metadata(slots), scaling=1.0)
    exact, mag = _exact(proj, x.contiguous(), y0[:, 1024:2048].contiguous(), slots)
    _check(yw[:, 1024:2048].contiguous(), y0[:, 1024:2048].contiguous(), exact, mag, slots, "strided")
    assert torch.equal(yw[:, :1024], y0[:, :1024]) and torch.equal(yw[:, 2048:], y0[:, 2048:])

    layer = LoRALinear(64, 48, bias=True, max_loras=2, max_lora_rank=8).cuda().to(torch.bfloat16)
    g = torch.Generator().manual_seed(3)
    with torch.no_grad():
        layer.weight.copy_(torch.randn(48, 64, generator=g) * 0.1)
        layer.bias.copy_(torch.randn(48, generator=g) * 0.1)
        for s in range(2):
            layer.set_slot_lora(s, (torch.randn(8, 64, generator=g) * 0.2).cuda(), (torch.randn(48, 8, generator=g) * 0.2).cuda(), 8, 0.5)
    x3 = torch.randn(3, 5, 64, generator=g).to(torch.bfloat16).cuda()
    slots = torch.tensor([0, 1, -1, 1, 0] * 3, dtype=torch.int32, device="cuda")
    set_lora_context(build_lora_context_from_token_to_slot(slots))
    with torch.no_grad():
        y3 = layer(x3)
        base = torch.nn.functional.linear(x3, layer.weight, layer.bias)
    assert y3.shape == (3, 5, 48)
    (want,) = oracle.fused_add_lora([base.reshape(15, 48).cpu()], x3.reshape(15, 64).cpu(), [layer.lora_A.detach().cpu()], [layer.lora_B.detach().cpu()],
                                    indices=slots.cpu(), scaling=1.0, accumulate=torch.float64)
    assert torch.allclose(y3.reshape(15, 48).cpu().float(), want.float(), rtol=RTOL, atol=ATOL)


# ---- low-level ops -------------------------------------------------------------------------------


def test_lora_shrink_known_answers():
    """reference tests/unit/test_lora_cuda.py:836-872 (K=160, r=8) and :875-911 (K=4096, r=1)."""
    from nanovllm_voxcpm_amd.lora_ops import lora_shrink

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")  # noqa: E731
    meta = (i32([0, 1, 0, 1]), i32([0, 2, 1, 3]), i32([2, 2, 0]), i32([0, 2, 4, 4]), i32([0, 1, -1]), False, 2)
    g = torch.Generator().manual_seed(8)
    for K, r, tol in ((160, 8, 5e-2), (4096, 1, 2e-1)):
        if K == 160:
            inputs = (torch.arange(4 * K, dtype=torch.float32).reshape(4, K) / 100).to(torch.float16).cuda()
        else:
            inputs = torch.randn(4, K, generator=g).to(torch.float16).cuda()
        lora_a = torch.randn(2, r, K, generator=g).to(torch.float16).cuda()
        out = torch.empty((1, 4, r), device="cuda", dtype=torch.float16)
        lora_shrink(inputs, [lora_a], out, *meta, 0.5)
        expected = torch.empty(4, r)
        for t, s in enumerate([0, 1, 0, 1]):
            expected[t] = torch.matmul(inputs[t].float().cpu(), lora_a[s].float().cpu().transpose(0, 1)) * 0.5
        assert torch.allclose(out.squeeze(0).float().cpu(), expected, atol=tol, rtol=tol)
        want = oracle.lora_shrink(inputs.cpu(), [lora_a.cpu()], torch.tensor([0, 1, 0, 1]), 0.5)
        assert torch.allclose(out.float().cpu(), want.float(), rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_lora_shrink_expand_against_oracle(dtype):
    from nanovllm_voxcpm_amd.lora_ops import LoRAKernelMeta, lora_expand, lora_shrink

    g = torch.Generator().manual_seed(12)
    T, K, r, L = 50, 96, 12, 5
    widths = [40, 24, 24]
    x = torch.randn(T, K, generator=g).to(dtype).cuda()
    a = [(torch.randn(L, r, K, generator=g) * 0.2).to(dtype).cuda() for _ in widths]
    b = [(torch.randn(L, n, r, generator=g) * 0.2).to(dtype).cuda() for n in widths]
    slots = torch.randint(-1, L, (T,), generator=g, dtype=torch.int32).cuda()
    meta = LoRAKernelMeta.make(L, T, "cuda")
    meta.prepare_tensors(slots)
    args = meta.meta_args(T, specialize_active_lora=True)
    tmp = torch.full((3, T, r), 7.0, dtype=dtype, device="cuda")
    lora_shrink(x, a, tmp, *args, 0.5)
    want_h = oracle.lora_shrink(x.cpu(), [t.cpu() for t in a], slots.cpu(), 0.5)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=RTOL, atol=ATOL)
    assert torch.allclose(tmp.cpu().float(), want_h.float(), **tol)
    assert torch.count_nonzero(tmp[:, slots < 0]) == 0
    out0 = torch.randn(T, 100, generator=g).to(dtype).cuda()
    for add in (False, True):
        out = out0.clone()
        lora_expand(tmp, b, out, *args, offset_start=8, add_inputs=add)
        want = oracle.lora_expand(tmp.cpu(), [t.cpu() for t in b], out0.cpu(), slots.cpu(), offset_start=8, add_inputs=add)
        assert torch.allclose(out.cpu().float(), want.float(), **tol)
        assert torch.equal(out[:, :8], out0[:, :8]) and torch.equal(out[:, 96:], out0[:, 96:])
        assert torch.equal(out[slots < 0], out0[slots < 0])
    # fp32 intermediate with 16-bit weights (the reference's CAST_TYPE case)
    if dtype != torch.float32:
        out = out0.clone()
        lora_expand(tmp.float(), b, out, *args, offset_start=8, add_inputs=True)
        want = oracle.lora_expand(tmp.float().cpu(), [t.cpu() for t in b], out0.cpu(), slots.cpu(), offset_start=8, add_inputs=True)
        assert torch.allclose(out.cpu().float(), want.float(), **tol)
    # no_lora_flag leaves the outputs alone
    untouched = tmp.clone()
    lora_shrink(x, a, tmp, args[0], args[1], args[2], args[3], args[4], True, 0, 0.5)
    assert torch.equal(tmp, untouched)


def test_backend_shrink_expand_helpers():
    backend = _backend()
    g = torch.Generator().manual_seed(2)
    x = torch.randn(9, 40, generator=g).cuda()
    a = torch.randn(6, 40, generator=g).cuda()
    b = torch.randn(14, 6, generator=g).cuda()
    h = backend.shrink(x, a)
    assert torch.allclose(h, torch.nn.functional.linear(x, a), rtol=1e-5, atol=1e-5)
    out = backend.expand(h, b, scaling=0.25)
    assert torch.allclose(out, torch.nn.functional.linear(h, b) * 0.25, rtol=1e-5, atol=1e-5)


# ---- slot install --------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_install_slot_is_bit_exact_with_torch(dtype):
    """One launch == zero slot, copy A[:rank], copy B[:, :rank] * scaling (reference layers/lora.py:395-417)."""
    from nanovllm_voxcpm_amd.layers.lora import LoRAMergedColumnParallelLinear, LoRARowParallelLinear

    g = torch.Generator().manual_seed(31)
    layer = LoRARowParallelLinear(72, 40, max_loras=3, max_lora_rank=16).to(dtype).cuda()
    with torch.no_grad():
        layer.lora_A.fill_(3.0)
        layer.lora_B.fill_(3.0)
    a_src = torch.randn(16, 72, generator=g).to(dtype).cuda()
    b_src = torch.randn(40, 16, generator=g).to(dtype).cuda()
    layer.set_slot_lora(1, a_src, b_src, effective_rank=10, scaling=0.37)
    want_a = torch.zeros(16, 72, dtype=dtype, device="cuda"); want_a[:10] = a_src[:10]
    want_b = torch.zeros(40, 16, dtype=dtype, device="cuda"); want_b[:, :10] = b_src[:, :10] * 0.37
    assert torch.equal(layer.lora_A[1], want_a) and torch.equal(layer.lora_B[1], want_b)
    assert torch.all(layer.lora_A[0] == 3.0) and torch.all(layer.lora_B[2] == 3.0)
    assert layer.effective_lora_rank.tolist() == [0, 10, 0] and layer._effective_lora_rank_values == [0, 10, 0]
    layer.clear_slot_lora(1)
    assert torch.count_nonzero(layer.lora_A[1]) == 0 and torch.count_nonzero(layer.lora_B[1]) == 0
    # fp32 payload into 16-bit buffers, host-resident payload, stacked targets
    merged = LoRAMergedColumnParallelLinear(24, [16, 8], max_loras=2, max_lora_rank=4).to(dtype).cuda()
    a3 = torch.randn(2, 4, 24, generator=g)
    b3 = [torch.randn(16, 4, generator=g), torch.randn(8, 4, generator=g)]
    merged.set_slot_lora(1, a3, b3, effective_rank=3, scaling=2.0)
    for pos in range(2):
        wa = torch.zeros(4, 24); wa[:3] = a3[pos, :3]
        wb = torch.zeros(b3[pos].size(0), 4); wb[:, :3] = b3[pos][:, :3] * 2.0
        assert torch.equal(merged.lora_A[pos, 1].cpu(), wa.to(dtype))
        assert torch.equal(getattr(merged, f"lora_B_{pos}")[1].cpu(), wb.to(dtype))


# ---- on-device metadata against the integer oracle ----------------------------------------------------


@pytest.mark.parametrize("T,L,p_neg", [(1, 1, 0.0), (7, 3, 0.5), (256, 32, 0.0), (300, 17, 0.3), (4096, 128, 0.1), (8192, 128, 0.0), (20000, 1024, 0.2), (513, 600, 0.0)])
def test_metadata_bit_exact_random(T, L, p_neg):
    from nanovllm_voxcpm_amd import _hip
    from nanovllm_voxcpm_amd.engine.graph_meta import copy_lora_domain_to_graph_vars, make_graph_domain_buffers
    from nanovllm_voxcpm_amd.lora_ops import LoRAKernelMeta, build_segment_plan
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, build_lora_context_from_token_to_slot

    rng = np.random.default_rng(T * 31 + L)
    slots = rng.integers(0, L, size=T)
    slots[rng.random(T) < p_neg] = -1
    if T > 4000:  # a few long segments
        slots[: T // 3] = slots[0]
    slots_l = [int(v) for v in slots]
    dev = torch.tensor(slots_l, dtype=torch.int32, device="cuda")
    s, a, c, o = meta_oracle.engine_layout(slots_l)

    ctx = build_lora_context_from_token_to_slot(dev, max_slots=L)
    if not a:
        assert ctx.no_lora_flag
    else:
        assert ctx.token_indices_sorted_by_slot.tolist() == s and ctx.active_slot_ids.tolist() == a
        assert ctx.num_tokens_per_slot.tolist() == c and ctx.slot_start_offsets.tolist() == o
        lazy = build_lora_context_from_token_to_slot(dev, max_slots=L, sync=False)
        cap = min(T, L)
        assert lazy.active_slot_ids.tolist() == a + [-1] * (cap - len(a))
        assert lazy.num_tokens_per_slot.tolist() == c + [0] * (cap - len(a))
        assert lazy.slot_start_offsets.tolist() == o + [0] * (cap - len(a))
        assert lazy.token_indices_sorted_by_slot[: len(s)].tolist() == s

    km = LoRAKernelMeta.make(L, T + 5, "cuda")
    km.prepare_tensors(dev)
    want = meta_oracle.kernel_meta_layout(slots_l, L)
    assert km.no_lora_flag is want["no_lora_flag"] and km.num_active_loras == want["num_active_loras"]
    assert km.active_lora_ids.tolist() == want["active_lora_ids"]
    assert km.num_tokens_per_lora.tolist() == want["num_tokens_per_lora"]
    assert km.lora_token_start_loc.tolist() == want["lora_token_start_loc"]
    if want["sorted_idx"] is not None:
        assert km.token_indices_sorted_by_lora_ids[:T].tolist() == want["sorted_idx"]
        assert km.token_lora_mapping[:T].tolist() == slots_l

    bufs = make_graph_domain_buffers(T + 9, L + 1, "cuda")
    copy_lora_domain_to_graph_vars(bufs, LoRAContext(token_to_slot=dev, no_lora_flag=not a))
    g = meta_oracle.graph_layout(slots_l, not a, T + 9, L + 1)
    for key, val in g.items():
        assert bufs[key].tolist() == val, key

    plan = build_segment_plan(dev, L)
    hdr = plan.header()
    short, long_small, long_big = meta_oracle.plan_tiles(slots_l, L)
    assert hdr[_hip.PLAN_MAGIC] == _hip.PLAN_MAGIC_VALUE and hdr[_hip.PLAN_NUM_TOKENS] == T and hdr[_hip.PLAN_MAX_SLOTS] == L
    assert hdr[_hip.PLAN_NUM_LORA_TOKENS] == len(s) and hdr[_hip.PLAN_NUM_ACTIVE] == len(a)
    assert hdr[_hip.PLAN_NO_LORA] == (0 if a else 1) and hdr[_hip.PLAN_BAD_SLOT] == 0
    assert hdr[_hip.PLAN_TILES_SHORT] == len(short) and hdr[_hip.PLAN_TILES_LONG_SMALL] == len(long_small)
    assert hdr[_hip.PLAN_TILES_LONG_BIG] == len(long_big) and hdr[_hip.PLAN_MAX_SEGMENT] == (max(c) if c else 0)
    ws = plan.workspace.tolist()
    r4 = lambda v: (v + 3) & ~3  # noqa: E731
    sorted_off = _hip.PLAN_HEADER_WORDS
    counts_off = sorted_off + r4(T)
    offsets_off = counts_off + r4(L + 1)
    small_off = (offsets_off + r4(L + 2) + 31) & ~31
    cap_small = ((T + 15) // 16 + min(L, T) + 7) & ~7
    big_off = small_off + _hip.SMALL_TILE_WORDS * cap_small
    cap_big = meta_oracle.big_tile_capacity(T, L)
    bigrows_off = big_off + 4 * cap_big
    slotrec_off = bigrows_off + 64 * cap_big
    cap_slotrec = (L + 7) & ~7
    over_off = slotrec_off + 32 * cap_slotrec
    cap_over = (T // 16 + 7) & ~7
    assert len(ws) == over_off + 32 * cap_over
    # the small tiles once more, by slot: a record per slot id, then the further tiles of every slot
    first, further = meta_oracle.plan_tiles_by_slot(slots_l, L)
    check = (0x4D4C5031 ^ T ^ (L << 20)) & 0xFFFFFFFF
    check = check - (1 << 32) if check >= 1 << 31 else check  # as the int32 word reads
    assert hdr[_hip.PLAN_TILES_OVER] == len(further) and hdr[_hip.PLAN_REJECTED] == 0
    assert len(further) <= T // 16

    def record(at):
        return ws[at : at + 32]

    for slot, (count, start) in enumerate(first):
        rec = record(slotrec_off + 32 * slot)
        assert rec[:4] == [slot, count, start, check]
        own = s[start : start + count]
        assert rec[4:20] == ([own[j % count] for j in range(16)] if count else [0] * 16) and rec[20:] == [0] * 12
    for slot in range(L, cap_slotrec):
        assert record(slotrec_off + 32 * slot) == [-1, 0, 0, check] + [0] * 28
    for q, (slot, start, count) in enumerate(further):
        rec = record(over_off + 32 * q)
        assert rec[:4] == [slot, count, start, check]
        own = s[start : start + count]
        assert rec[4:20] == [own[j % count] for j in range(16)] and rec[20:] == [0] * 12
    for q in range(len(further), cap_over):
        assert record(over_off + 32 * q) == [-1, 0, 0, check] + [0] * 28
    # both lists hold the same tiles
    assert sorted([(sl, st, c) for sl, (c, st) in enumerate(first) if c] + further) == sorted(short + long_small)
    assert ws[sorted_off : sorted_off + len(s)] == s
    dense = [0] * (L + 1)
    for slot, n in zip(a, c):
        dense[slot + 1] = n
    assert ws[counts_off : counts_off + L + 1] == dense
    assert ws[offsets_off : offsets_off + L + 2] == [0] + list(np.cumsum(dense))
    for q, (slot, start, count) in enumerate(short + long_small):
        rec = ws[small_off + 32 * q : small_off + 32 * (q + 1)]
        assert rec[:4] == [slot, count, start, 0]
        own = s[start : start + count]
        assert rec[4:20] == [own[j % count] for j in range(16)] and rec[20:] == [0] * 12  # cyclic repeats past the count
    place = meta_oracle.big_tile_places(long_big, T, L)
    assert len(set(place)) == len(place) and all(0 <= q < cap_big for q in place)
    assert [tuple(ws[big_off + 4 * q : big_off + 4 * q + 3]) for q in place] == long_big
    assert all(tuple(ws[big_off + 4 * q : big_off + 4 * q + 3]) == (-1, 0, 0) for q in set(range(cap_big)) - set(place))  # places without a tile
    for q, (slot, start, count) in zip(place, long_big):  # the tile's tokens, then zeros (a valid row to read)
        own = s[start : start + count]
        assert ws[bigrows_off + 64 * q : bigrows_off + 64 * (q + 1)] == own + [0] * (64 - count)


def test_metadata_flags_bad_slot_ids():
    from nanovllm_voxcpm_amd import _hip
    from nanovllm_voxcpm_amd.lora_ops import build_segment_plan

    plan = build_segment_plan(torch.tensor([0, 5, 1, -1], dtype=torch.int32, device="cuda"), 2)
    hdr = plan.header()
    assert hdr[_hip.PLAN_BAD_SLOT] == 1 and hdr[_hip.PLAN_NUM_LORA_TOKENS] == 2


# ---- graph capture -----------------------------------------------------------------------------------


def test_graph_capture_replays_follow_new_slots_inputs_and_weights():
    """A layer forward captured once is replayed with new activations, new slot ids (same
    buffers) and a slot installed after capture; every replay is checked against an eager run
    (reference tests/unit/test_lora_cuda.py:224-281, 618-667)."""
    from nanovllm_voxcpm_amd.engine.graph_meta import make_graph_domain_buffers, set_graph_lora_contexts
    from nanovllm_voxcpm_amd.layers.lora import LoRAQKVParallelLinear
    from nanovllm_voxcpm_amd.utils.context import LORA_DOMAINS, LoRAContext, reset_lora_context, set_lora_context

    torch.manual_seed(0)
    L, rank, T = 4, 16, 24
    layer = LoRAQKVParallelLinear(256, 64, 4, 2, max_loras=L, max_lora_rank=rank).cuda().to(torch.bfloat16)
    g = torch.Generator().manual_seed(77)
    with torch.no_grad():
        layer.weight.copy_(torch.randn(layer.weight.shape, generator=g) * 0.05)

    def install(slot, seed):
        gg = torch.Generator().manual_seed(seed)
        a = torch.randn(3, rank, 256, generator=gg) * 0.1
        b = [torch.randn(n, rank, generator=gg) * 0.1 for n in (256, 128, 128)]
        layer.set_slot_lora(slot, a, b, effective_rank=rank, scaling=1.0)

    for s in range(3):
        install(s, 10 + s)
    graph_vars = {"lora_domains": {d: make_graph_domain_buffers(T, L + 1, "cuda") for d in LORA_DOMAINS}}
    x_buf = torch.zeros(T, 256, dtype=torch.bfloat16, device="cuda")
    out_buf = torch.zeros(T, 512, dtype=torch.bfloat16, device="cuda")
    empty = LoRAContext(no_lora_flag=True)

    def stage(slots):
        ctx = LoRAContext(token_to_slot=torch.tensor(slots, dtype=torch.int32, device="cuda"), no_lora_flag=False)
        set_graph_lora_contexts(graph_vars, {LORA_DOMAINS[0]: ctx, LORA_DOMAINS[1]: empty, LORA_DOMAINS[2]: empty})

    def eager(x, slots):
        reset_lora_context()
        set_lora_context(LoRAContext(token_to_slot=torch.tensor(slots, dtype=torch.int32, device="cuda"), no_lora_flag=False))
        with torch.no_grad():
            return layer(x).clone()

    slots0 = [0] * T
    stage(slots0)
    with torch.no_grad():
        out_buf.copy_(layer(x_buf))  # warm-up outside capture, same context object
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out_buf.copy_(layer(x_buf))

    rng = np.random.default_rng(4)
    for step in range(4):
        slots = [int(v) for v in rng.integers(-1, 3 if step < 2 else 4, size=T)]
        if step == 2:
            install(3, 99)  # adapter admitted after capture
        x = torch.randn(T, 256, generator=g).to(torch.bfloat16).cuda()
        want = eager(x, slots)          # eager work between replays
        torch.cuda.synchronize()
        stage(slots)                    # refresh the fixed buffers in place
        x_buf.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_buf, want), f"replay {step} differs from eager"


@pytest.mark.parametrize("name,tokens,rank", [("down", 256, 16), ("gate_up", 1500, 64), ("down", 1500, 32)])
def test_graph_replays_of_the_shared_and_the_two_launch_forms(name, tokens, rank):
    """Backend call captured once (K = 4096 at decode size: producer and consumer workgroups
    exchanging partial sums through the scratch; 1500 tokens: the two-launch form; in both the
    scratch is allocated and initialised inside the capture) and replayed with new activations, base outputs and slot ids in
    the same buffers; every replay is checked against the fp64 evaluation and against an eager
    call on the same inputs, with eager work and synchronisations between the replays."""
    from nanovllm_voxcpm_amd import synthetic

    print(f"graph {name} T={tokens} r={rank}", flush=True)
    slots_n = 8
    proj = _make(name, slots_n, rank, torch.bfloat16, seed=600 + rank)
    x_buf = torch.zeros(tokens, proj.k, dtype=torch.bfloat16, device="cuda")
    y_buf = torch.zeros(tokens, sum(proj.widths), dtype=torch.bfloat16, device="cuda")
    s_buf = torch.zeros(tokens, dtype=torch.int32, device="cuda")
    backend = _backend()
    blocks = list(y_buf.split(proj.widths, dim=-1))
    packed = y_buf if len(blocks) > 1 else None

    def call(meta):
        backend.add_lora(blocks, x_buf, proj.a, proj.b, indices=s_buf, metadata=meta, scaling=1.0, y_packed=packed)

    call(_metadata(s_buf))  # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(_metadata(s_buf))  # a fresh metadata object: the plan launch is part of the graph

    g = torch.Generator().manual_seed(61)
    for step in range(4):
        x, y0 = synthetic.make_activations(tokens, proj.k, sum(proj.widths), torch.bfloat16, seed=610 + step, device="cuda")
        if tokens <= 1024:
            slots = torch.randint(-1, slots_n, (tokens,), generator=g, dtype=torch.int32)
        else:
            slots, _ = synthetic.prefill_slots(12, slots_n, seed=620 + step, min_len=40, max_len=200)
            slots = torch.nn.functional.pad(slots, (0, max(0, tokens - slots.numel())), value=-1)[:tokens]
        slots = slots.cuda()
        x_buf.copy_(x); y_buf.copy_(y0); s_buf.copy_(slots)
        call(_metadata(s_buf))  # eager call on the same buffers
        eager = y_buf.clone()
        torch.cuda.synchronize()
        y_buf.copy_(y0)
        graph.replay()
        torch.cuda.synchronize()
        exact, mag = _exact(proj, x, y0, slots)
        _check(y_buf, y0, exact, mag, slots, f"graph/{name}/T{tokens}/step{step}")
        assert torch.equal(y_buf, eager), f"replay {step} differs from the eager call"


def test_slot_major_grid_takes_three_slices_that_lie_far_apart():
    """The three-slice kernel gets the second and third slice's weight pointers as 40-bit offsets
    (units of 16 bytes) from the first one's.  The slices of a projection are allocations of their
    own; here the first slice's buffers lie at the start of a 36 GiB allocation and the others' at
    its end, so the offsets do not fit 32 bits.  The result is the oracle's and, bit for bit, the
    tile-major grid's."""
    from nanovllm_voxcpm_amd import synthetic

    print("slot-major qkv, slices 36 GiB apart", flush=True)
    free, _ = torch.cuda.mem_get_info()
    if free < (48 << 30):
        pytest.skip("needs 48 GiB of free device memory")
    L, rank, T = 8, 16, 64
    base = _make("qkv", L, rank, torch.bfloat16, seed=1400)
    arena = torch.empty(36 << 30, dtype=torch.uint8, device="cuda")
    cursor = [arena.numel()]

    def at_the_end(t):  # a copy of t in the arena, carved from its end (256-byte aligned)
        nbytes = (t.numel() * t.element_size() + 255) & ~255
        cursor[0] -= nbytes
        view = arena[cursor[0] : cursor[0] + t.numel() * t.element_size()].view(t.dtype).view(t.shape)
        view.copy_(t)
        return view

    def at_the_start(t, offset):
        view = arena[offset : offset + t.numel() * t.element_size()].view(t.dtype).view(t.shape)
        view.copy_(t)
        return view

    a0 = at_the_start(base.a[0], 0)
    b0 = at_the_start(base.b[0], (base.a[0].numel() * 2 + 255) & ~255)
    proj = synthetic.ProjectionWeights("qkv", base.k, list(base.widths), [a0, at_the_end(base.a[1]), at_the_end(base.a[2])],
                                       [b0, at_the_end(base.b[1]), at_the_end(base.b[2])])
    gaps = [proj.a[i].data_ptr() - proj.a[0].data_ptr() for i in (1, 2)] + [proj.b[i].data_ptr() - proj.b[0].data_ptr() for i in (1, 2)]
    assert min(gaps) > (32 << 30)
    x, y0 = synthetic.make_activations(T, proj.k, sum(proj.widths), torch.bfloat16, seed=1401, device="cuda")
    slots = synthetic.decode_slots(T, L, seed=1402).cuda()
    got = _apply("slot", proj, x, y0.clone(), slots)
    exact, mag = _exact(proj, x, y0, slots)
    _check(got, y0, exact, mag, slots, "slot-major/qkv/far apart")
    assert torch.equal(got, _apply("mfma", proj, x, y0.clone(), slots))
    # and with the later slices in front of the first one (negative offsets)
    back = synthetic.ProjectionWeights("qkv", base.k, list(base.widths), [proj.a[1], a0, proj.a[2]], [proj.b[1], b0, proj.b[2]])
    back.widths = [base.widths[1], base.widths[0], base.widths[2]]
    y1 = torch.randn(T, sum(back.widths), generator=torch.Generator().manual_seed(1403)).to(torch.bfloat16).cuda()
    got = _apply("slot", back, x, y1.clone(), slots)
    exact, mag = _exact(back, x, y1, slots)
    _check(got, y1, exact, mag, slots, "slot-major/qkv/far apart, first slice last in memory")
    torch.cuda.synchronize()
    del proj, back, a0, b0, arena
    torch.cuda.empty_cache()
