"""The entry point that allocates nothing (``mlora_add_lora_static``) against the regular one.

Both are called through the C-ABI binding on the same seeded inputs: first a batch whose long
segments take the two-launch form (the rank-r intermediate passes through the scratch), then,
straight after it on the same stream, a smaller batch.  The regular entry point is given a
caller-owned workspace of the same size as the library's static array, so both make the same
choices and the outputs have to be bit-identical; the larger batch is also held to the oracle at
the stated bf16 tolerance.  A size that does not fit the static array must be refused before any
launch.
"""

import pytest
import torch

from oracle import lora_apply as oracle

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3  # bf16 outputs, fp32 accumulation


def _run(static, proj, x, y0, slots, workspace):
    from nanovllm_voxcpm_amd import _hip
    from nanovllm_voxcpm_amd.lora_ops.segment_meta import build_segment_plan

    plan = build_segment_plan(slots, proj.a[0].size(0)).workspace
    y = y0.clone()
    cols, col = [], 0
    for n in proj.widths:
        cols.append(col)
        col += n
    _hip.add_lora(y, x, proj.a, proj.b, cols, slots, plan, 1.0, _hip.FORM_AUTO,
                  None if static else workspace, static_scratch=static)
    return y


@pytest.mark.parametrize("name,rank", [("gate_up", 64), ("down", 16)])
def test_static_scratch_entry_matches_the_regular_entry(name, rank):
    from nanovllm_voxcpm_amd import _hip, synthetic

    print(f"no-alloc entry {name} r={rank}", flush=True)
    dev = "cuda"
    proj = synthetic.make_projection(name, 6, rank, torch.bfloat16, seed=70 + rank, device=dev)
    workspace = torch.empty(_hip.STATIC_SCRATCH_BYTES, dtype=torch.uint8, device=dev)
    _hip.workspace_init(workspace)  # as every caller-owned workspace is, once, after allocation
    outs = []
    for tokens, seed in ((1500, 71), (130, 72)):  # two calls in a row, the second one smaller
        x, y0 = synthetic.make_activations(tokens, proj.k, sum(proj.widths), torch.bfloat16, seed=seed, device=dev)
        g = torch.Generator().manual_seed(seed)
        slots = torch.randint(-1, 6, (tokens,), generator=g, dtype=torch.int32)
        slots[: tokens // 2] = 2  # one long segment, the rest short ones
        slots = slots.to(dev)
        got = _run(True, proj, x, y0, slots, None)
        ref = _run(False, proj, x, y0, slots, workspace)
        outs.append((got, ref, x, y0, slots))
    torch.cuda.synchronize()
    for got, ref, x, y0, slots in outs:
        assert torch.equal(got, ref), "static-scratch entry and regular entry disagree"
        assert not torch.equal(got, y0)
        live = slots >= 0
        assert torch.equal(got[~live], y0[~live])
    got, _, x, y0, slots = outs[0]
    want = oracle.fused_add_lora(list(y0.cpu().split(proj.widths, dim=-1)), x.cpu(), [a.cpu() for a in proj.a],
                                 [b.cpu() for b in proj.b], indices=slots.cpu(), scaling=1.0, accumulate=torch.float64)
    assert torch.allclose(got.cpu().float(), torch.cat(want, dim=-1).float(), rtol=RTOL, atol=ATOL)


def test_static_scratch_entry_refuses_what_does_not_fit():
    from nanovllm_voxcpm_amd import _hip

    dev = "cuda"
    tokens, rank, slices = 40000, 64, 2  # 40000 x 2 x 64 x 4 bytes = 20.5 MB > 16 MiB
    x = torch.zeros(tokens, 128, dtype=torch.bfloat16, device=dev)
    y = torch.zeros(tokens, 16, dtype=torch.bfloat16, device=dev)
    a = [torch.zeros(1, rank, 128, dtype=torch.bfloat16, device=dev) for _ in range(slices)]
    b = [torch.zeros(1, 8, rank, dtype=torch.bfloat16, device=dev) for _ in range(slices)]
    slots = torch.zeros(tokens, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="exceed the static scratch"):
        _hip.add_lora(y, x, a, b, [0, 8], slots, None, 1.0, static_scratch=True)


def test_static_scratch_entry_under_graph_capture_after_a_warm_up_call():
    """The address of the library's scratch is looked up on the first call on a device, which must
    not happen inside a capture (the library refuses that with a clear error): one call with no
    tokens, outside any capture, is the warm-up.  After it the entry point can be captured; every
    replay gives the bits of the eager call."""
    from nanovllm_voxcpm_amd import _hip, synthetic
    from nanovllm_voxcpm_amd.lora_ops.segment_meta import build_segment_plan

    dev = "cuda"
    proj = synthetic.make_projection("o", 6, 16, torch.bfloat16, seed=75, device=dev)
    tokens = 96
    x, y0 = synthetic.make_activations(tokens, proj.k, sum(proj.widths), torch.bfloat16, seed=76, device=dev)
    g = torch.Generator().manual_seed(77)
    slots = torch.randint(-1, 6, (tokens,), generator=g, dtype=torch.int32).to(dev)
    plan = build_segment_plan(slots, 6).workspace
    empty = torch.zeros(0, proj.k, dtype=torch.bfloat16, device=dev)
    _hip.add_lora(y0[:0], empty, proj.a, proj.b, [0], slots[:0], None, 1.0, static_scratch=True)  # warm-up: no tokens, no launch
    eager = y0.clone()
    _hip.add_lora(eager, x, proj.a, proj.b, [0], slots, plan, 1.0, _hip.FORM_AUTO, None, static_scratch=True)
    torch.cuda.synchronize()
    y = y0.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _hip.add_lora(y, x, proj.a, proj.b, [0], slots, plan, 1.0, _hip.FORM_AUTO, None, static_scratch=True,
                      stream=_hip.current_stream_handle(x.device))
    for _ in range(3):
        y.copy_(y0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager)
