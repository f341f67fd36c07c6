"""Benchmark of the fused multi-LoRA apply on one MI355X.

Default workload (BASELINE.json configs[1], "decode BGMV bf16"): one decode step of a 24-layer
decoder — 256 tokens (one per sequence), 32 resident adapters of rank 16, adapter ids uniform,
LoRA applied to the stacked q|k|v [1024|256|256], o [1024->1024], gate|up [1024->2x4096] and
down [4096->1024] projections of every layer.  A "step" is the LoRA work of that step: one
on-device metadata build plus 24 x 4 fused shrink+expand calls, issued through the same backend
entry (`LoRABackend.add_lora`) the LoRA linears call.  Every layer owns its weights and its
activation buffers (about 0.75 GB in total), so a step streams from HBM and not from the 256 MB
last-level cache.

Prints ONE JSON line.  `value` = algorithmic bytes of a step / time of a step, inputs resident
in HBM, the step replayed as a captured graph (decode runs under graph replay in the serving
engine).  `roofline` is quoted for the kernel that does the work of the step: algorithmic bytes
of an average launch / average launch time.  `cpu_baseline` times the reference's torch
formulation (per-token F.linear loop) of one layer of the same workload on the host cores.

`--workload prefill` (configs[2]: 16 sequences of 64..1024 tokens, 8 adapters of rank 64, a
quarter of the sequences without adapter) and `--workload mixed` (configs[3]: 2 x 2048-token
chunks + 4096 decodes, 128 adapters of ranks {8,16,32,64} padded to 64, Zipf popularity) time the
same 24 x 4 calls on those batches; they are measurement aids, the driver runs the default.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (ROOT, ROOT / "nanovllm-voxcpm_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_TFLOPS = 2500.0  # MI355X dense bf16, published
NUM_LAYERS = 24
ORDER = ("qkv", "o", "gate_up", "down")

WORKLOADS = {
    "decode": dict(slots=32, rank=16, distinct_layers=24,
                   text="decode BGMV bf16 (BASELINE configs[1]): 256 tokens, 32 adapters, rank 16, "
                        "qkv/o/gate_up/down x 24 layers, per-layer weights and activations"),
    "prefill": dict(slots=8, rank=64, distinct_layers=4,
                    text="prefill SGMV bf16 (BASELINE configs[2]): 16 sequences of 64..1024 tokens, 8 adapters, "
                         "rank 64, 25% of sequences without adapter, qkv/o/gate_up/down x 24 layers"),
    "backbone": dict(slots=32, rank=32, distinct_layers=24,
                     text="synthetic backbone bf16 (BASELINE configs[4]): 24 layers, hidden 1024, 16 q / 2 kv heads, "
                          "SwiGLU 4096, 64 decode streams, context U[128,2048], 32 rank-32 adapters on all linears"),
    "mixed": dict(slots=128, rank=64, distinct_layers=4,
                  text="mixed bf16 (BASELINE configs[3]): 2 x 2048-token chunks + 4096 decodes, 128 adapters of "
                       "ranks {8,16,32,64} padded to 64, Zipf(1.1), qkv/o/gate_up/down x 24 layers"),
}


def algorithmic_bytes(k: int, widths: list[int], t_lora: int, used_slots: int, rank: int, num_tokens: int,
                      rank_sum: int | None = None) -> int:
    """bf16 bytes one fused call has to move: x rows, the A and B slices of the slots in use,
    y read and written once, plus the int32 slot ids; the rank-r intermediate counts as zero.
    ``rank_sum``: sum of the true ranks of the slots in use when adapters of lower rank sit in
    rank-``rank`` buffers and the kernels are told so (rows beyond a slot's rank are not moved)."""
    s, n = len(widths), sum(widths)
    ranks = used_slots * rank if rank_sum is None else rank_sum
    return 2 * (t_lora * k + ranks * s * k + ranks * n + 2 * t_lora * n) + 4 * num_tokens


def algorithmic_flops(k: int, widths: list[int], t_lora: int, rank: int, token_rank_sum: int | None = None) -> int:
    """``token_rank_sum``: sum over the tokens of their slot's true rank, when it is below ``rank``."""
    return 2 * (t_lora * rank if token_rank_sum is None else token_rank_sum) * (len(widths) * k + sum(widths))


def build_workload(name: str, device: str, rank: int | None = None, sequences: int = 0, slot_ids: int = 0):
    """Per-layer (projection weights, x, y) for the distinct layers of the workload and the
    batch's slot vector.  Layers beyond the distinct ones reuse buffers round-robin (the distinct
    set alone exceeds the 256 MB last-level cache)."""
    import torch

    from nanovllm_voxcpm_amd import synthetic

    spec = WORKLOADS[name]
    rank = rank or spec["rank"]
    num_slots = max(slot_ids, spec["slots"]) if name == "decode" else spec["slots"]  # decode: buffers with more slot ids than adapters in use
    if name == "decode":
        slots = synthetic.decode_slots(256, spec["slots"], seed=7)
        ranks = None
    elif name == "prefill":
        slots, _ = synthetic.prefill_slots(sequences or 16, spec["slots"], seed=301)
        ranks = None
    else:
        slots = synthetic.mixed_slots(seed=402)
        ranks = synthetic.heterogeneous_ranks(spec["slots"], seed=400)
    num_tokens = slots.numel()
    distinct = []
    for layer in range(spec["distinct_layers"]):
        entry = {}
        for j, proj_name in enumerate(ORDER):
            proj = synthetic.make_projection(proj_name, num_slots, rank, torch.bfloat16,
                                             seed=1000 + 16 * layer + j, device=device, true_ranks=ranks)
            x, y = synthetic.make_activations(num_tokens, proj.k, sum(proj.widths), torch.bfloat16,
                                              seed=5000 + 16 * layer + j, device=device)
            entry[proj_name] = (proj, x, y)
        distinct.append(entry)
    layers = [distinct[i % len(distinct)] for i in range(NUM_LAYERS)]
    eff = torch.tensor(ranks, dtype=torch.int32, device=device) if ranks is not None else None
    return layers, slots.to(device), eff


def make_step(layers, slots, form: str, only: str | None = None, eff=None):
    """Returns step(): metadata build + every fused apply of one step, via the backend.  ``eff``:
    per-slot true ranks, handed to the backend as the LoRA linears do for padded buffers."""
    from nanovllm_voxcpm_amd.lora import HipLoRABackend, LoRAMetadata

    backend = HipLoRABackend(form)
    status = backend.availability()
    if not status.available:
        raise RuntimeError(f"HIP LoRA backend unavailable: {status.reason}")
    names = list(only) if isinstance(only, (tuple, list)) else [only] if only else list(ORDER)
    calls = []
    for entry in layers:
        for name in names:
            proj, x, y = entry[name]
            blocks = list(y.split(proj.widths, dim=-1))
            calls.append((blocks, x, proj.a, proj.b, y if len(blocks) > 1 else None))

    def step():
        # a new metadata object per step, as the engine installs a new context per step:
        # the first call builds the segment plan on the device, the others reuse it
        meta = LoRAMetadata(slots, None, None, None, None, False, 0)
        for blocks, x, a, b, packed in calls:
            backend.add_lora(blocks, x, a, b, indices=slots, metadata=meta, scaling=1.0, y_packed=packed, effective_rank=eff)

    step.backend = backend
    return step, len(calls)


def time_region(fn, iters: int) -> float:
    """Milliseconds per call of fn, HIP events on torch's current stream (the stream every
    kernel of fn is launched on), synchronised on both sides."""
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def capture(step):
    import torch

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    return graph


def cpu_baseline(layers, slots, rank: int, budget_s: float = 20.0) -> dict:
    """The reference's torch LoRA computation on the host: per-token F.linear(F.linear(x_t, A[s]),
    B[s]) accumulate (oracle.per_token_add_lora), fp32, one layer of the same workload, all host
    threads.  Reported in the metric's unit: algorithmic bytes of what was run / time."""
    import torch

    from oracle import lora_apply as oracle

    threads = torch.get_num_threads()
    entry = layers[0]
    slots_cpu = slots.cpu()
    num_tokens = slots_cpu.numel()
    work = []
    for name in ORDER:
        proj, x, y = entry[name]
        work.append((proj, x.cpu().float(), y.cpu().float(), [a.cpu().float() for a in proj.a], [b.cpu().float() for b in proj.b]))
    used = int(torch.unique(slots_cpu[slots_cpu >= 0]).numel())
    t_lora = int((slots_cpu >= 0).sum())
    layer_bytes = sum(algorithmic_bytes(p.k, p.widths, t_lora, used, rank, num_tokens) for p, *_ in work)

    def one_layer():
        for proj, x, y, a, b in work:
            views = list(y.split(proj.widths, dim=-1))
            oracle.per_token_add_lora(views, x, a, b, indices=slots_cpu, scaling=1.0, y_packed=y)

    def timed(fn, budget):
        fn()  # warm-up
        samples = []
        t_end = time.perf_counter() + budget
        while len(samples) < 3 or (time.perf_counter() < t_end and len(samples) < 20):
            t0 = time.perf_counter()
            fn()
            samples.append(time.perf_counter() - t0)
        samples.sort()
        return samples[len(samples) // 2], len(samples)

    med, runs = timed(one_layer, budget_s * 0.5)
    times = [0.0] * runs

    # two more views of the same layer, a few seconds each: the loop on one thread, and the
    # vectorised restatement (gather + two batched matmuls per slice) on all threads
    def one_layer_vectorised():
        for proj, x, y, a, b in work:
            for a_i, b_i in zip(a, b):
                oracle.fused_delta(x, a_i, b_i, slots_cpu, 1.0)

    vec_med, _ = timed(one_layer_vectorised, budget_s * 0.2)
    torch.set_num_threads(1)
    try:
        one_med, _ = timed(one_layer, budget_s * 0.3)
    finally:
        torch.set_num_threads(threads)
    # the model string as the host reports it (a virtual machine may report the family name only:
    # family / model / stepping numbers are appended, they identify the part)
    model, ids = "", {}
    try:
        for line in Path("/proc/cpuinfo").read_text().splitlines():
            if not line.strip():
                break  # first processor only
            key, _, val = line.partition(":")
            key = key.strip()
            if key == "model name":
                model = val.strip()
            elif key in ("cpu family", "model", "stepping"):
                ids[key] = val.strip()
    except OSError:
        pass
    if ids:
        model = f"{model} (family {ids.get('cpu family', '?')} model {ids.get('model', '?')} stepping {ids.get('stepping', '?')})".strip()
    return {
        "value": round(layer_bytes / med / 1e9, 4),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"1 of {NUM_LAYERS} layers of the same step (4 projections, {num_tokens} tokens, rank {rank}), fp32, "
                  f"per-token torch loop, median of {len(times)} runs",
        "us_per_layer": round(med * 1e6, 1),
        "variants_us_per_layer": {"per_token_loop_1_thread": round(one_med * 1e6, 1),
                                  f"gather_bmm_{threads}_threads": round(vec_med * 1e6, 1)},
        "us_per_step_extrapolated": round(med * 1e6 * NUM_LAYERS, 1),
        "cpu_model": model,
        "host_cpus": os.cpu_count(),
    }


def measure_backbone(steps: int, warmup: int) -> dict:
    """BASELINE configs[4]: decode-step latency of a synthetic 24-layer decoder (hidden 1024, 16 query /
    2 KV heads of 64, SwiGLU 4096, RMSNorm; 64 streams with context lengths U[128, 2048]; 32 rank-32
    adapters on all linears) with the LoRA kernels against the same step with LoRA disabled."""
    import torch

    from nanovllm_voxcpm_amd.backbone import MiniDecoder
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, reset_lora_context, set_lora_context

    device = "cuda:0"
    streams, adapters, rank = 64, 32, 32
    model = MiniDecoder(max_loras=adapters, rank=rank).to(device=device, dtype=torch.bfloat16)
    model.init_random(seed=500, adapters=adapters, rank=rank)
    g = torch.Generator().manual_seed(501)
    positions = torch.randint(128, 2049, (streams,), generator=g).to(device)
    slots = torch.randint(0, adapters, (streams,), generator=g, dtype=torch.int32).to(device)
    x = torch.randn(streams, model.hidden, generator=g).to(torch.bfloat16).to(device)
    caches = model.make_cache(streams, 2049, torch.bfloat16, device, seed=502)

    def timed(lora_on: bool):
        reset_lora_context()
        if lora_on:
            set_lora_context(LoRAContext(token_to_slot=slots, no_lora_flag=False))
        with torch.inference_mode():
            for _ in range(2):
                out = model(x, caches, positions)
            torch.cuda.synchronize()
            eager = time_region(lambda: model(x, caches, positions), 3)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out = model(x, caches, positions)
            for _ in range(warmup):
                graph.replay()
            ms = time_region(graph.replay, steps)
        reset_lora_context()
        return ms, eager, out.float().clone()

    off_ms, off_eager, y_off = timed(False)
    on_ms, on_eager, y_on = timed(True)
    return {
        "workload": WORKLOADS["backbone"]["text"], "streams": streams, "adapters": adapters, "rank": rank, "launch": "graph replay",
        "steps": steps, "us_per_step": round(on_ms * 1e3, 2), "us_per_step_lora_off": round(off_ms * 1e3, 2),
        "us_lora_cost": round((on_ms - off_ms) * 1e3, 2), "us_lora_cost_per_call": round((on_ms - off_ms) * 1e3 / (4 * NUM_LAYERS), 3),
        "lora_overhead_pct": round(100 * (on_ms - off_ms) / off_ms, 2),
        "us_per_step_eager": {"lora_on": round(on_eager * 1e3, 1), "lora_off": round(off_eager * 1e3, 1)},
        "lora_changes_output": bool((y_on - y_off).abs().max().item() > 0),
    }


def run_backbone(args) -> None:
    r = measure_backbone(args.steps, args.warmup)
    print(json.dumps({
        "metric": "decode-step latency of the synthetic backbone, LoRA kernels on vs LoRA disabled (us), 1 GPU",
        "value": r["us_per_step"], "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["us_per_step"] / 1e3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {k: r[k] for k in ("workload", "streams", "adapters", "rank", "launch")},
        **{k: r[k] for k in ("us_per_step_lora_off", "us_lora_cost", "us_lora_cost_per_call", "lora_overhead_pct", "us_per_step_eager",
                             "lora_changes_output")},
    }))


KERNELS = {
    "decode": "slot_kernel3<bf16,16> (qkv) + slot_kernel<bf16,16> (o, gate_up, down)",
    "prefill": "wide_kernel<bf16,64> (qkv, o) + sgmv_shrink_kernel<bf16,64> + sgmv_expand_kernel<bf16,64> (gate_up, down)",
    "mixed": "wide_kernel<bf16,64> (qkv, o) + sgmv_shrink_kernel<bf16,64> + sgmv_expand_kernel<bf16,64> (gate_up, down)",
}


def kernel_sources_sha256() -> str:
    """Hash of the kernel sources: measured counter figures are quoted only for the sources they
    were measured on."""
    import hashlib

    h = hashlib.sha256()
    csrc = ROOT / "nanovllm-voxcpm_amd" / "csrc"
    for path in sorted(list(csrc.glob("*.hip")) + list(csrc.glob("*.h")) + [ROOT / "include" / "mlora.h"]):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()


def recorded_traffic(workload: str):
    """HBM bytes per average launch of ``workload`` from the rocprofv3 counter runs summarised in
    profiles/roofline.json, or None when that file was measured on other kernel sources."""
    try:
        rec = json.loads((ROOT / "profiles" / "roofline.json").read_text())
    except (OSError, ValueError):
        return None
    if rec.get("kernel_sources_sha256") != kernel_sources_sha256():
        return None
    return rec.get("traffic_bytes_per_launch", {}).get(workload)


def measure_workload(name: str, device: str, form: str, steps: int, warmup: int, *, only=None, rank=0, hot_layers=0, eager=False,
                     per_projection=True, rank_vector=True, sequences=0, slot_ids=0) -> tuple[dict, tuple]:
    """Time one workload: its step replayed as a captured graph (or eagerly), per-projection steps,
    bytes, flops and the roofline object.  Returns (result, (layers, slots, rank, step))."""
    import torch

    spec = WORKLOADS[name]
    rank = rank or spec["rank"]
    layers, slots, eff = build_workload(name, device, rank, sequences, slot_ids)
    if not rank_vector:
        eff = None
    if hot_layers > 0:
        layers = [layers[i % hot_layers] for i in range(NUM_LAYERS)]
    step, launches = make_step(layers, slots, form, only, eff)

    num_tokens = slots.numel()
    used_ids = torch.unique(slots[slots >= 0])
    used = int(used_ids.numel())
    t_lora = int((slots >= 0).sum())
    rank_sum = token_rank_sum = None
    if eff is not None:  # adapters of lower rank in rank-`rank` buffers, and the kernels are told
        rank_sum = int(eff[used_ids.long()].sum())
        token_rank_sum = int(eff[slots[slots >= 0].long()].sum())
    names = list(only) if isinstance(only, (tuple, list)) else [only] if only else list(ORDER)
    shapes = {n: layers[0][n][0] for n in names}
    per_proj = {n: algorithmic_bytes(p.k, p.widths, t_lora, used, rank, num_tokens, rank_sum) for n, p in shapes.items()}
    per_proj_flops = {n: algorithmic_flops(p.k, p.widths, t_lora, rank, token_rank_sum) for n, p in shapes.items()}
    step_bytes = NUM_LAYERS * sum(per_proj.values())
    step_flops = NUM_LAYERS * sum(per_proj_flops.values())

    for _ in range(2):
        step()
    torch.cuda.synchronize()
    eager_ms = time_region(step, max(3, min(steps, 20)))
    if eager:
        runner = step
    else:
        graph = capture(step)
        runner = graph.replay
    for _ in range(warmup):
        runner()
    ms = time_region(runner, steps)

    # per-projection time: the same step restricted to one projection (24 launches)
    per_proj_us = {}
    if per_projection and not isinstance(only, str) and not eager:
        for n in names:
            sub, cnt = make_step(layers, slots, form, n, eff)
            g = capture(sub)
            for _ in range(2):
                g.replay()
            per_proj_us[n] = round(time_region(g.replay, max(3, steps // 4)) * 1e3 / cnt, 3)

    value = step_bytes / (ms * 1e-3) / 1e9
    calls = launches
    launch_bytes = step_bytes / calls
    call_us = ms * 1e3 / calls
    default_shape = form == "auto" and not only and not hot_layers and rank == spec["rank"] and not sequences and not slot_ids
    result = {
        "value": round(value, 2),
        "ms_per_step": round(ms, 5),
        "config": {
            "workload": spec["text"] if rank == spec["rank"] else spec["text"] + f" -- run at rank {rank} instead",
            "tokens": num_tokens, "tokens_with_adapter": t_lora, "adapters": spec["slots"], "adapters_in_batch": used,
            "slot_ids_of_the_buffers": max(slot_ids, spec["slots"]) if name == "decode" else spec["slots"],
            "rank": rank, "layers": NUM_LAYERS, "projections": names, "form": form,
            "launch": "eager" if eager else "graph replay",
            "distinct_layer_buffers": hot_layers or spec["distinct_layers"],
        },
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "us_per_step": round(ms * 1e3, 2),
        "us_per_step_eager": round(eager_ms * 1e3, 2),
        "algorithmic_bytes_per_step": step_bytes,
        "algorithmic_flops_per_step": step_flops,
        "tflops": round(step_flops / (ms * 1e-3) / 1e12, 2),
        "pct_of_mfma_bf16_peak": round(100 * step_flops / (ms * 1e-3) / 1e12 / MFMA_BF16_TFLOPS, 3),
        "calls_per_step": calls,
        "algorithmic_bytes_per_call_by_projection": per_proj,
        "us_per_call_by_projection": per_proj_us,
        "gbs_by_projection": {n: round(per_proj[n] / (per_proj_us[n] * 1e-6) / 1e9, 1) for n in per_proj_us},
        "roofline": {
            "kernel": "bgmv_kernel<bf16>" if form == "bgmv" else KERNELS[name],
            "bound": "hbm",
            # algorithmic bytes of an average call / time of an average call inside the replayed
            # step (HIP events around the replays on the stream the kernels run on)
            "achieved": round(value, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(value / HBM_PEAK_GBS, 4),
            # HBM bytes per average call from the rocprofv3 counter runs (profiles/roofline.json),
            # quoted only when the kernel sources are the ones those runs measured
            "traffic": recorded_traffic(name) if default_shape else None,
            "bytes_per_call": round(launch_bytes),
            "us_per_call": round(call_us, 3),
        },
    }
    if eff is not None:
        result["config"]["true_rank_sum_of_adapters_in_batch"] = rank_sum
        result["config"]["mean_true_rank_per_token"] = round(token_rank_sum / max(t_lora, 1), 2)
    return result, (layers, slots, rank, step)


def measure_unfused(layers, slots, name: str = "qkv") -> dict:
    """The two-call form (lora_shrink into an fp32 intermediate, then lora_expand with add_inputs)
    on one projection of the decode workload, beside the fused call on the same buffers: a graph
    of the 24 layers' calls each, microseconds per projection call."""
    import torch

    from nanovllm_voxcpm_amd.lora_ops import lora_expand, lora_shrink

    proj0 = layers[0][name][0]
    n_slices, rank = len(proj0.widths), proj0.a[0].size(1)
    h = torch.zeros((n_slices, slots.numel(), rank), dtype=torch.float32, device=slots.device)

    def two_calls():
        for entry in layers:
            proj, x, y = entry[name]
            lora_shrink(x, list(proj.a), h, slots, None, None, None, None, False, 0, 1.0)
            lora_expand(h, list(proj.b), y, slots, None, None, None, None, False, 0, offset_start=0, add_inputs=True)

    fused, calls = make_step(layers, slots, "auto", only=name)
    out = {}
    for key, fn in (("us_per_call_shrink_then_expand", two_calls), ("us_per_call_fused", fused)):
        graph = capture(fn)
        for _ in range(3):
            graph.replay()
        out[key] = round(time_region(graph.replay, 20) * 1e3 / calls, 2)
    out["projection"] = name
    return out


def measure_long_form_latency(layers, slots) -> dict:
    """What a call of the two-launch long-segment form costs before it moves any data to speak of:
    the prefill step's 96 calls (same buffers, same grids) on a batch in which no token has an
    adapter slot (both launches find nothing to do) and on one in which a single token has one (one
    workgroup per launch walks the whole chain: record, token rows, operands, multiply, store).
    Microseconds per call, graph replay."""
    import torch

    out = {}
    none = torch.full_like(slots, -1)
    one = none.clone()
    one[0] = 0
    for key, batch in (("us_per_call_no_token_has_a_slot", none), ("us_per_call_one_token_has_a_slot", one)):
        step, calls = make_step(layers, batch, "sgmv")
        graph = capture(step)
        for _ in range(3):
            graph.replay()
        out[key] = round(time_region(graph.replay, 10) * 1e3 / calls, 2)
    return out


def measure_floor(device: str, step_bytes: int, calls: int) -> dict:
    """What bounds a step of `calls` dependent launches on this machine, measured in this run:
    a replayed graph of as many kernels that do nothing (one wavefront each, then the grid of a
    decode launch), the same number of real launches on a plan without any token to serve (every
    workgroup fetches its tile record and leaves), and plain streams over a buffer of half a
    step's bytes (read-modify-write as y is touched, and read-only)."""
    import torch

    from nanovllm_voxcpm_amd import _hip, synthetic
    from nanovllm_voxcpm_amd.lora import HipLoRABackend, LoRAMetadata

    def graph_of(fn):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        for _ in range(3):
            g.replay()
        return time_region(g.replay, 20) * 1e3

    tiny = graph_of(lambda: [_hip.probe_launch(0, grid=(1, 1, 1), threads=64) for _ in range(calls)]) / calls
    grid = graph_of(lambda: [_hip.probe_launch(0, grid=(8, 6, 6), threads=512) for _ in range(calls)]) / calls

    # the real launches of a decode step on a batch in which no token has an adapter slot
    backend = HipLoRABackend()
    none = torch.full((256,), -1, dtype=torch.int32, device=device)
    work = []
    for j, name in enumerate(ORDER):
        proj = synthetic.make_projection(name, 32, 16, torch.bfloat16, seed=90 + j, device=device)
        x, y = synthetic.make_activations(256, proj.k, sum(proj.widths), torch.bfloat16, seed=95 + j, device=device)
        blocks = list(y.split(proj.widths, dim=-1))
        work.append((blocks, x, proj.a, proj.b, y if len(blocks) > 1 else None))

    def empty_plan_step():
        meta = LoRAMetadata(none, None, None, None, None, False, 0)
        for i in range(calls):
            blocks, x, a, b, packed = work[i % len(work)]
            backend.add_lora(blocks, x, a, b, indices=none, metadata=meta, scaling=1.0, y_packed=packed)

    empty_plan = graph_of(empty_plan_step) / calls

    half = (step_bytes // 2 + 255) & ~255
    buf = torch.zeros(half // 2, dtype=torch.bfloat16, device=device)
    out = {"launches": calls, "us_per_empty_launch_one_wavefront": round(tiny, 3), "us_per_empty_launch_decode_grid": round(grid, 3),
           "us_per_real_launch_on_a_plan_without_tokens": round(empty_plan, 3)}
    for kind, key, factor in ((1, "stream_read_modify_write_gbs", 2), (2, "stream_read_only_gbs", 1)):
        for _ in range(2):
            _hip.probe_launch(kind, buf)
        ms = time_region(lambda: _hip.probe_launch(kind, buf), 10)
        out[key] = round(factor * half / (ms * 1e-3) / 1e9, 1)
    # the step if every launch cost what a launch without tokens costs and its bytes moved at the
    # rate of the read-modify-write stream, with no overlap between the two
    out["us_per_step_floor_launches_plus_stream"] = round(calls * empty_plan + step_bytes / (out["stream_read_modify_write_gbs"] * 1e3), 1)
    return out


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="decode", choices=sorted(WORKLOADS))
    ap.add_argument("--form", default="auto", help="kernel family: auto | bgmv | mfma | slot | split | sgmv | wide | fused | token")
    ap.add_argument("--only", default=None, choices=ORDER, help="restrict the step to one projection (profiling)")
    ap.add_argument("--eager", action="store_true", help="time eager launches instead of graph replay")
    ap.add_argument("--slot-ids", type=int, default=0,
                    help="decode workload: weight buffers with this many slot ids (the batch still uses 32 adapters): what slot ids "
                         "nobody uses cost the slot-major grid (MLORA_SLOT_MAX_SLOTS bounds where AUTO takes it)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip what the default run adds after the headline: the prefill, mixed and backbone steps and the floor")
    ap.add_argument("--floor", action="store_true", help="print only the floor measurements (launch costs and stream rates)")
    ap.add_argument("--rank", type=int, default=0,
                    help="the decode or prefill workload at another adapter rank (buffers of that rank); 0 = the workload's own")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device tensor copy, as the known-size reference "
                         "that rocprof byte counters of the same run are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; every box in this pool has one (use --gpus 1)")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm GPU visible")
    device = "cuda:0"
    torch.cuda.set_device(0)
    if args.workload == "backbone":
        run_backbone(args)
        return
    if args.floor:
        print(json.dumps({"floor": measure_floor(device, 918650880, 4 * NUM_LAYERS)}))
        return

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)  # 256 MiB read + 256 MiB written
        torch.cuda.synchronize()
        del src, dst

    heavy = args.workload != "decode"
    steps = args.steps if not heavy else max(3, min(args.steps, 30))
    warmup = args.warmup if not heavy else max(1, min(args.warmup, 3))
    rank = args.rank if args.workload in ("decode", "prefill") else 0
    res, (layers, slots, rank, step) = measure_workload(args.workload, device, args.form, steps, warmup, only=args.only, rank=rank,
                                                        eager=args.eager, slot_ids=args.slot_ids if args.workload == "decode" else 0)
    out = {
        "metric": "multi-LoRA shrink+expand HBM GB/s (% peak); us per decode step, 1 GPU",
        "value": res["value"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
    }
    out.update({k: v for k, v in res.items() if k not in ("value", "ms_per_step")})
    out["launches_per_step"] = res["calls_per_step"] * (2 if args.workload != "decode" else 1) + 1

    # waits of the split form that ran out during everything above (0 in a healthy run: a consumer
    # workgroup that gives up computes its intermediate itself, which is correct but slow)
    from nanovllm_voxcpm_amd import _hip

    torch.cuda.synchronize()
    out["split_waits_run_out"] = sum(
        int(buf[: 4 * (_hip.WORKSPACE_TIMEOUTS_WORD + 1)].view(torch.int32)[_hip.WORKSPACE_TIMEOUTS_WORD].item())
        for buf in step.backend.scratch_buffers())

    default_run = args.workload == "decode" and args.form == "auto" and not args.only and not args.eager and not args.rank and not args.slot_ids
    if default_run and not args.no_extras:
        # After the headline (outside its timed region): what one launch costs here and what a
        # stream reaches here, and the other configurations of the benchmark, a few replays each.
        try:  # (launches of known cost come from the diagnostic variant of the library)
            out["floor"] = measure_floor(device, res["algorithmic_bytes_per_step"], res["calls_per_step"])
        except RuntimeError as exc:
            out["floor"] = {"unavailable": str(exc)}
        extra = {}
        for name in ("prefill", "mixed"):
            r, (wl_layers, wl_slots, _, _) = measure_workload(name, device, "auto", 5, 2, per_projection=True)
            extra[name] = {k: r[k] for k in ("config", "us_per_step", "us_per_step_eager", "value", "pct_of_hbm_peak", "tflops",
                                             "pct_of_mfma_bf16_peak", "algorithmic_bytes_per_step", "us_per_call_by_projection", "roofline")}
            extra[name]["unit"] = "GB/s"
            if name == "prefill":
                extra[name]["latency"] = measure_long_form_latency(wl_layers, wl_slots)
            del wl_layers, wl_slots
            torch.cuda.empty_cache()
        # the reference's own default LoRA shape (max_lora_rank 32, targets q / k / v / o only:
        # nanovllm_voxcpm/models/voxcpm/config.py:87-90) on the same decode batch
        r, _ = measure_workload("decode", device, "auto", 50, 10, only=("qkv", "o"), rank=32)
        extra["reference_default"] = {k: r[k] for k in ("config", "us_per_step", "us_per_step_eager", "value", "pct_of_hbm_peak",
                                                        "algorithmic_bytes_per_step", "calls_per_step", "us_per_call_by_projection",
                                                        "gbs_by_projection")}
        extra["reference_default"]["unit"] = "GB/s"
        torch.cuda.empty_cache()
        extra["backbone"] = measure_backbone(10, 3)
        extra["unfused_ops"] = measure_unfused(layers, slots)
        torch.cuda.empty_cache()
        out["extra"] = extra
    if not args.no_cpu_baseline and args.workload == "decode":
        out["cpu_baseline"] = cpu_baseline(layers, slots, rank, budget_s=10.0)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
