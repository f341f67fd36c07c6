"""CPU-only checks: the C-ABI library loads and exports what include/mlora.h declares, the
ctypes structs match the C layout, arguments are rejected before any launch, and the host
logic of the backend / layers behaves like the reference's (error text included)."""

import ctypes as C
import re
import subprocess
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "mlora.h"


def _declared_functions() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mlora_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from nanovllm_voxcpm_amd import _hip

    lib = _hip.load()
    declared = _declared_functions()
    assert declared and set(declared) == set(_hip.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.mlora_abi_version() == int(re.search(r"#define MLORA_ABI_VERSION (\d+)", HEADER.read_text()).group(1)) == 4
    assert "gfx950" in _hip.build_info()


def test_measurement_aids_live_in_the_diagnostic_variant_only():
    """include/mlora.h is the product's C-ABI; what include/mlora_diag.h declares is exported by
    the diagnostic variant of the library (the knob reload, which the tests of one process need,
    by the product library too) and nothing else of it by the product library."""
    from nanovllm_voxcpm_amd import _hip

    diag_header = HEADER.with_name("mlora_diag.h")
    text = re.sub(r"/\*.*?\*/", "", diag_header.read_text(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(mlora_[a-z_]+)\s*\(", text)))
    assert set(declared) == set(_hip.DIAG_EXPORTS)
    assert not set(declared) & set(_declared_functions())
    lib = _hip.load()
    assert hasattr(lib, "mlora_reload_knobs")
    assert not hasattr(lib, "mlora_probe_launch") and not hasattr(lib, "mlora_trace_set")
    diag = _hip.load_diag()
    for name in _hip.EXPORTS + _hip.DIAG_EXPORTS:
        assert hasattr(diag, name), name


def test_ctypes_structs_match_the_c_layout(tmp_path):
    """Compile a probe against the header with the host compiler and compare sizeof / offsetof."""
    from nanovllm_voxcpm_amd import _hip

    structs = {
        "MloraSlice": _hip.MloraSlice,
        "MloraAddArgs": _hip.MloraAddArgs,
        "MloraShrinkArgs": _hip.MloraShrinkArgs,
        "MloraExpandArgs": _hip.MloraExpandArgs,
        "MloraMetaArgs": _hip.MloraMetaArgs,
        "MloraInstallArgs": _hip.MloraInstallArgs,
    }
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "mlora.h"', "int main(void) {"]
    for name, st in structs.items():
        lines.append(f'  printf("{name} %zu\\n", sizeof({name}));')
        for field, _ in st._fields_:
            lines.append(f'  printf("{name}.{field} %zu\\n", offsetof({name}, {field}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "probe.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "probe"
    subprocess.run(["gcc", "-std=c11", f"-I{HEADER.parent}", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    got = dict(line.split() for line in out.strip().splitlines())
    for name, st in structs.items():
        assert int(got[name]) == C.sizeof(st), name
        for field, _ in st._fields_:
            assert int(got[f"{name}.{field}"]) == getattr(st, field).offset, f"{name}.{field}"
    assert _hip.MAX_SLICES == 8 and _hip.TILE_SMALL == 16 and _hip.TILE_BIG == 64 and _hip.SEGMENT_THRESHOLD == 16
    text = HEADER.read_text()
    for macro, value in (("MLORA_MAX_SLICES", 8), ("MLORA_MAX_SLOTS", _hip.MAX_SLOTS), ("MLORA_MAX_RANK", _hip.MAX_RANK),
                         ("MLORA_TILE_SMALL", 16), ("MLORA_SMALL_TILE_WORDS", _hip.SMALL_TILE_WORDS), ("MLORA_BIG_TILE_WORDS", _hip.BIG_TILE_WORDS), ("MLORA_TILE_BIG", 64), ("MLORA_SEGMENT_THRESHOLD", 16),
                         ("MLORA_PLAN_HEADER_WORDS", _hip.PLAN_HEADER_WORDS), ("MLORA_FORM_SPLIT", _hip.FORM_SPLIT),
                         ("MLORA_FORM_SLOT", _hip.FORM_SLOT), ("MLORA_PLAN_TILES_OVER", _hip.PLAN_TILES_OVER),
                         ("MLORA_PLAN_REJECTED", _hip.PLAN_REJECTED), ("MLORA_PLAN_MAX_SEGMENT", _hip.PLAN_MAX_SEGMENT)):
        assert re.search(rf"#define {macro} {value}\b", text), macro
    assert re.search(r"#define MLORA_WORKSPACE_HEAD_BYTES \(16384 \+ \(4 << 20\) \+ \(64 << 10\)\)", text) and _hip.WORKSPACE_HEAD_BYTES == 16384 + (4 << 20) + (64 << 10)
    assert re.search(r"#define MLORA_STATIC_SCRATCH_BYTES \(16u << 20\)", text) and _hip.STATIC_SCRATCH_BYTES == 16 << 20


def test_arguments_are_rejected_before_any_launch():
    from nanovllm_voxcpm_amd import _hip

    lib = _hip.load()
    assert lib.mlora_add_lora(None) == -1 and b"NULL args" in lib.mlora_last_error()
    args = _hip.MloraAddArgs()
    args.num_tokens = -1
    assert lib.mlora_add_lora(C.byref(args)) == -1
    args = _hip.MloraAddArgs()
    args.num_tokens, args.k, args.r, args.num_slots, args.num_slices, args.dtype = 4, 8, 8, 2, 9, 2
    assert lib.mlora_add_lora(C.byref(args)) == -3 and b"slices" in lib.mlora_last_error()
    args.num_slices, args.dtype = 1, 7
    assert lib.mlora_add_lora(C.byref(args)) == -1 and b"dtype" in lib.mlora_last_error()
    args.dtype, args.r = 2, 1000
    assert lib.mlora_add_lora(C.byref(args)) == -3
    args.r, args.num_slots = 8, 5000
    assert lib.mlora_add_lora(C.byref(args)) == -3
    args.num_slots = 2  # valid sizes, NULL tensors
    assert lib.mlora_add_lora(C.byref(args)) == -1 and b"NULL tensor" in lib.mlora_last_error()
    # rows that would overlap or run past their stride (dummy addresses: rejected before any use)
    args.x, args.y, args.token_to_slot = 0x1000, 0x2000, 0x3000
    args.x_stride, args.y_stride = 8, 8
    args.slices[0].a, args.slices[0].b, args.slices[0].n, args.slices[0].y_col = 0x4000, 0x5000, 16, 0
    assert lib.mlora_add_lora(C.byref(args)) == -1 and b"y row stride" in lib.mlora_last_error()
    args.y_stride, args.x_stride = 16, 4
    assert lib.mlora_add_lora(C.byref(args)) == -1 and b"x row stride" in lib.mlora_last_error()
    args.num_tokens = 0  # nothing to do is success
    assert lib.mlora_add_lora(C.byref(args)) == 0
    meta = _hip.MloraMetaArgs()
    meta.max_slots = 5000
    assert lib.mlora_meta_build(C.byref(meta)) == -3
    meta.max_slots, meta.num_tokens = 4, 3
    assert lib.mlora_meta_build(C.byref(meta)) == -1  # NULL token_to_slot with tokens
    assert lib.mlora_shrink(None) == -1 and lib.mlora_expand(None) == -1 and lib.mlora_install_slot(None) == -1
    # slot install: a slot beyond the buffers and source rows shorter than what they carry are refused
    inst = _hip.MloraInstallArgs()
    inst.a_dst, inst.b_dst, inst.a_src, inst.b_src = 0x1000, 0x2000, 0x3000, 0x4000
    inst.k, inst.n, inst.r, inst.rank, inst.num_slots, inst.slot = 64, 32, 16, 8, 4, 4
    inst.a_src_stride, inst.b_src_stride, inst.dtype, inst.src_dtype = 64, 8, 2, 0
    assert lib.mlora_install_slot(C.byref(inst)) == -1 and b"outside the 4 slots" in lib.mlora_last_error()
    inst.slot, inst.a_src_stride = 3, 32
    assert lib.mlora_install_slot(C.byref(inst)) == -1 and b"row strides" in lib.mlora_last_error()
    inst.a_src_stride, inst.rank = 64, 17
    assert lib.mlora_install_slot(C.byref(inst)) == -1 and b"bad sizes" in lib.mlora_last_error()
    # workspace initialisation: alignment and the minimum size are checked before any launch
    assert lib.mlora_workspace_init(0x1010, 1 << 22, None) == -1 and b"aligned" in lib.mlora_last_error()
    assert lib.mlora_workspace_init(0x1000, 4096, None) == -1 and b"MLORA_WORKSPACE_HEAD_BYTES" in lib.mlora_last_error()
    assert lib.mlora_add_workspace_bytes(256, 3, 16, 2) == _hip.WORKSPACE_HEAD_BYTES + 4 * 256 * 3 * 16 * 4
    assert lib.mlora_plan_workspace_bytes(256, 32) == 4 * _hip.plan_workspace_words(256, 32) > 0
    assert lib.mlora_plan_workspace_bytes(-1, 2) == 0
    # the plan's layout as documented: header, sorted indices, dense counts and offsets, small tiles, big
    # tiles and their row lists, then a 128-byte record per slot id and per further tile
    def words(t, l):
        r4 = lambda v: (v + 3) & ~3  # noqa: E731
        small_off = (16 + r4(t) + r4(l + 1) + r4(l + 2) + 31) & ~31
        cap_small = ((t + 15) // 16 + min(l, t) + 7) & ~7
        most = t // 64 + min(l, t)  # big tiles at most; an eighth of them + about the root of that + 2 fit each of eight blocks
        root = next(v for v in range(1, most + 2) if 8 * v * v >= most)
        cap_big = (most + 8 * (root + 2) + 31) & ~31
        return small_off + 32 * cap_small + (4 + 64) * cap_big + 32 * ((l + 7) & ~7) + 32 * ((t // 16 + 7) & ~7)
    for t, l in ((256, 32), (1, 1), (8192, 128), (20000, 1024), (15, 600)):
        assert lib.mlora_plan_workspace_bytes(t, l) == 4 * words(t, l), (t, l)


def test_no_gpu_means_unavailable_and_loud():
    """Without a GPU the probed backend refuses every compute call; nothing falls back to the host."""
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from nanovllm_voxcpm_amd import lora
    from nanovllm_voxcpm_amd.utils.context import build_lora_context_from_token_to_slot

    lora._PROBED_BACKEND = None
    backend = lora.get_backend()
    assert isinstance(backend, lora._UnavailableBackend)
    assert lora.is_available() is False and "GPU" in lora.get_availability().reason
    with pytest.raises(RuntimeError):
        lora.assert_available()
    x = torch.zeros(2, 8)
    with pytest.raises(RuntimeError):
        backend.add_lora([x], x, [x], [x], indices=None, metadata=None, scaling=1.0)
    with pytest.raises(RuntimeError):
        backend.shrink(x, x)
    with pytest.raises(RuntimeError):
        backend.expand(x, x, scaling=1.0)
    with pytest.raises(RuntimeError, match="no host fallback"):
        build_lora_context_from_token_to_slot(torch.tensor([0, 1], dtype=torch.int32))
    # a forced HIP backend with host tensors must refuse as well
    meta = lora.LoRAMetadata(torch.zeros(2, dtype=torch.int32), None, None, None, None, False, 0)
    a, b = torch.zeros(1, 4, 8), torch.zeros(1, 8, 4)
    with pytest.raises(RuntimeError, match="no host fallback"):
        lora.HipLoRABackend().add_lora([torch.zeros(2, 8)], x, [a], [b], indices=meta.token_to_slot, metadata=meta, scaling=1.0)


def test_missing_library_is_reported(monkeypatch, tmp_path):
    from nanovllm_voxcpm_amd import _hip

    monkeypatch.setenv("MLORA_LIBRARY", str(tmp_path / "absent.so"))
    monkeypatch.setattr(_hip, "_LIB", None)
    monkeypatch.setattr(_hip, "_LOAD_ERROR", None)
    with pytest.raises(RuntimeError, match="not built"):
        _hip.load()
    assert "not built" in _hip.load_error()


def test_add_lora_argument_validation_matches_reference_errors():
    """reference nanovllm_voxcpm/lora.py:264-289"""
    from nanovllm_voxcpm_amd.lora import HipLoRABackend, LoRAMetadata

    backend = HipLoRABackend()
    x = torch.zeros(2, 4)
    a, b, y = torch.zeros(1, 2, 4), torch.zeros(1, 3, 2), torch.zeros(2, 3)
    meta = LoRAMetadata(torch.zeros(2, dtype=torch.int32), None, None, None, None, False, 0)
    idx = meta.token_to_slot
    assert backend.add_lora([], x, [], [], indices=idx, metadata=meta, scaling=1.0) == []
    with pytest.raises(ValueError, match="aligned y/lora_a/lora_b slice lists"):
        backend.add_lora([y], x, [a, a], [b], indices=idx, metadata=meta, scaling=1.0)
    with pytest.raises(RuntimeError, match="LoRA metadata must be prepared by the model runner"):
        backend.add_lora([y], x, [a], [b], indices=idx, metadata=None, scaling=1.0)
    with pytest.raises(ValueError, match="contiguous lora_a"):
        backend.add_lora([y], x, [torch.zeros(1, 4, 2).transpose(1, 2)], [b], indices=idx, metadata=meta, scaling=1.0)
    with pytest.raises(ValueError, match="contiguous lora_b"):
        backend.add_lora([y], x, [a], [torch.zeros(1, 2, 3).transpose(1, 2)], indices=idx, metadata=meta, scaling=1.0)
    with pytest.raises(ValueError, match="y_packed must be 2D"):
        backend.add_lora([y], x, [a], [b], indices=idx, metadata=meta, scaling=1.0, y_packed=torch.zeros(1, 2, 3))
    # no_lora_flag returns before touching the device
    quiet = LoRAMetadata(idx, None, None, None, None, True, 0)
    assert backend.add_lora([y], x, [a], [b], indices=idx, metadata=quiet, scaling=1.0)[0] is y
    with pytest.raises(ValueError, match="unknown LoRA kernel form"):
        HipLoRABackend("fast")
    assert meta.as_kernel_metadata(1)[0].numel() == 1 and meta.as_kernel_metadata(1)[5] is False


class _CountingBackend:
    def __init__(self):
        self.calls = []

    def availability(self):
        from nanovllm_voxcpm_amd.lora import LoRAAvailability

        return LoRAAvailability(True)

    def add_lora(self, y_slices, x, a, b, *, indices, metadata, scaling, y_packed=None):
        self.calls.append(dict(n=len(y_slices), packed=y_packed is not None, scaling=scaling, metadata=metadata, indices=indices))
        return list(y_slices)


def test_layer_gating_and_call_shapes():
    """reference nanovllm_voxcpm/layers/lora.py:78-113 (gates), :340-382, :546-586, :722-742 (calls)."""
    from nanovllm_voxcpm_amd.layers import lora as L
    from nanovllm_voxcpm_amd.lora import set_backend_for_testing
    from nanovllm_voxcpm_amd.utils.context import LoRAContext, reset_lora_context, set_lora_context

    spy = _CountingBackend()
    set_backend_for_testing(spy)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)  # noqa: E731
    qkv = L.LoRAQKVParallelLinear(8, 2, 2, 1, max_loras=2, max_lora_rank=2)
    merged = L.LoRAMergedColumnParallelLinear(8, [4, 4], max_loras=2, max_lora_rank=2)
    partial = L.LoRAQKVParallelLinear(8, 2, 2, 1, lora_targets=["q", "v"], max_loras=2, max_lora_rank=2)
    row = L.LoRARowParallelLinear(8, 4, max_loras=2, max_lora_rank=2)
    plain = L.LoRALinear(8, 4, max_loras=2, max_lora_rank=2)
    off = L.LoRALinear(8, 4)
    layers = [qkv, merged, partial, row, plain]
    for m in layers + [off]:
        with torch.no_grad():
            m.weight.zero_()
            if m.bias is not None:
                m.bias.zero_()
    x = torch.ones(3, 8)
    # no context, empty context, no_lora_flag, empty slot vector: base output, no backend call
    for ctx in (None, LoRAContext(), LoRAContext(token_to_slot=i32([0, 0, 0]), no_lora_flag=True), LoRAContext(token_to_slot=i32([]), no_lora_flag=False)):
        reset_lora_context()
        if ctx is not None:
            set_lora_context(ctx)
        for m in layers:
            m(x)
    assert spy.calls == []
    # slots in use but every slot empty in the module: skipped from the host mirrors
    set_lora_context(LoRAContext(token_to_slot=i32([0, 1, -1]), active_slot_ids=i32([0, 1]), no_lora_flag=False))
    for m in layers:
        m(x)
    assert spy.calls == []
    for m in layers:
        nt = len(getattr(m, "lora_targets", [])) or None
        a = torch.ones(nt, 2, 8) if nt else torch.ones(2, 8)
        if nt:
            b = [torch.ones(getattr(m, f"lora_B_{t}").size(1), 2) for t in m.lora_targets]
        else:
            b = torch.ones(m.lora_B.size(1), 2)
        m.validate_slot_lora_payload(a, b, 2, 1.0)
        m.set_slot_lora(1, a, b, 2, 1.0)
    for m in layers:
        m(x)
    assert [c["n"] for c in spy.calls] == [3, 2, 2, 1, 1]
    assert [c["packed"] for c in spy.calls] == [True, True, False, False, False]
    assert all(c["scaling"] == 1.0 for c in spy.calls)            # alpha/r lives in B
    assert len({id(c["metadata"]) for c in spy.calls}) == 1       # one metadata object per step
    assert spy.calls[0]["indices"].dtype == torch.int32
    # a context installed again drops the cached metadata
    set_lora_context(LoRAContext(token_to_slot=i32([0, 1, -1]), no_lora_flag=False))
    plain(x)
    assert spy.calls[-1]["metadata"] is not spy.calls[0]["metadata"]
    off(x)
    assert len(spy.calls) == 6
    # 3-D input is flattened for the call and restored
    set_lora_context(LoRAContext(token_to_slot=i32([1] * 6), no_lora_flag=False))
    assert plain(torch.ones(2, 3, 8)).shape == (2, 3, 4)
    with pytest.raises(RuntimeError, match="token_to_slot length does not match flattened input rows: token_to_slot=6 rows=3"):
        plain(x)
    assert [type(m) for m in L.iter_lora_modules(torch.nn.ModuleList(layers + [off]))] == [type(m) for m in layers]
    assert set(L.get_lora_state_dict(plain)) == {"lora_A", "lora_B"}


def test_slot_payload_validation_and_bookkeeping():
    """reference nanovllm_voxcpm/layers/lora.py:170-181, 419-450, 776-797"""
    from nanovllm_voxcpm_amd.layers import lora as L

    plain = L.LoRALinear(4, 3, max_loras=2, max_lora_rank=2)
    with pytest.raises(ValueError, match="exceeds max_lora_rank=2"):
        plain.set_slot_lora(0, torch.ones(3, 4), torch.ones(3, 3), 3, 1.0)
    with pytest.raises(ValueError, match="effective_rank must be > 0"):
        plain.validate_slot_lora_payload(torch.ones(2, 4), torch.ones(3, 2), 0, 1.0)
    with pytest.raises(ValueError, match="must be finite"):
        plain.validate_slot_lora_payload(torch.ones(2, 4), torch.ones(3, 2), 1, float("inf"))
    with pytest.raises(ValueError, match="expects tensor lora_b"):
        plain.validate_slot_lora_payload(torch.ones(2, 4), [torch.ones(3, 2)], 1, 1.0)
    with pytest.raises(ValueError, match="Expected lora_a input dim 4, got 5"):
        plain.validate_slot_lora_payload(torch.ones(2, 5), torch.ones(3, 2), 1, 1.0)
    with pytest.raises(ValueError, match="Expected lora_b output dim 3, got 7"):
        plain.validate_slot_lora_payload(torch.ones(2, 4), torch.ones(7, 2), 1, 1.0)
    with pytest.raises(ValueError, match="does not enable LoRA"):
        L.LoRALinear(4, 3).validate_slot_lora_payload(torch.ones(2, 4), torch.ones(3, 2), 1, 1.0)
    qkv = L.LoRAQKVParallelLinear(4, 2, 2, 1, max_loras=1, max_lora_rank=2)
    with pytest.raises(ValueError, match="expects lora_b to be a list"):
        qkv.validate_slot_lora_payload(torch.ones(3, 2, 4), torch.ones(4, 2), 1, 1.0)
    with pytest.raises(ValueError, match="Target 'k' expects output dim 2, got 4"):
        qkv.validate_slot_lora_payload(torch.ones(3, 2, 4), [torch.ones(4, 2), torch.ones(4, 2), torch.ones(2, 2)], 1, 1.0)
    merged = L.LoRAMergedColumnParallelLinear(4, [6, 2], max_loras=1, max_lora_rank=2)
    with pytest.raises(ValueError, match="Target 1 expects output dim 2, got 6"):
        merged.validate_slot_lora_payload(torch.ones(2, 2, 4), [torch.ones(6, 2), torch.ones(6, 2)], 1, 1.0)
    # scale folded into B once, rank padding zero, host mirrors kept
    plain.set_slot_lora(1, torch.full((2, 4), 3.0), torch.full((3, 2), 2.0), effective_rank=1, scaling=0.5)
    assert plain.lora_A[1].tolist() == [[3.0] * 4, [0.0] * 4]
    assert plain.lora_B[1].tolist() == [[1.0, 0.0]] * 3
    assert plain._effective_lora_rank_values == [0, 1] and plain._lora_scaling_values == [0.0, 0.5]
    assert plain.effective_lora_rank.tolist() == [0, 1] and plain._active_rank(1) == 1 and plain._slot_scaling(1) == 0.5
    plain.clear_slot_lora(1)
    assert torch.count_nonzero(plain.lora_A) == 0 and torch.count_nonzero(plain.lora_B) == 0
    assert plain._effective_lora_rank_values == [0, 0]
    # single-adapter checkpoint loaders (slot 0)
    qkv.load_lora_A(torch.ones(1, 4), "k")
    assert qkv.lora_A[1, 0, 0].tolist() == [1.0] * 4 and qkv._effective_lora_rank_values[0] == 1
    qkv.lora_B_k.weight_loader(qkv.lora_B_k, torch.full((2, 1), 4.0))
    assert qkv.lora_B_k[0, :, 0].tolist() == [4.0, 4.0]
    with pytest.raises(ValueError, match="exceeds max_lora_rank"):
        qkv.lora_B_k.weight_loader(qkv.lora_B_k, torch.ones(2, 3))
    qkv.reset_lora_parameters()
    assert torch.count_nonzero(qkv.lora_A) == 0 and torch.count_nonzero(qkv.lora_B_k) == 0


def test_batch_plan_host_side():
    from nanovllm_voxcpm_amd.engine.lora_manager import build_lora_batch_plan_from_token_to_slot, expand_token_to_slot

    slots = expand_token_to_slot([0, -1, 0], [2, 1, 1])
    assert slots == [0, 0, -1, 0]  # reference tests/unit/test_lora_runtime.py:86
    plan = build_lora_batch_plan_from_token_to_slot({7: 0}, slots)
    assert plan.active_slot_ids == [0] and plan.num_lora_tokens == 3
    with pytest.raises(ValueError, match="same length"):
        expand_token_to_slot([0], [1, 2])


def test_repo_has_no_product_import_of_the_oracle():
    pkg = ROOT / "nanovllm-voxcpm_amd"
    for path in pkg.rglob("*.py"):
        text = path.read_text()
        assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), path
    assert "oracle" not in sys.modules or True


def test_batch_plan_takes_the_six_reference_fields():
    """reference nanovllm_voxcpm/engine/lora_manager.py:67-75, 380: positional construction"""
    from nanovllm_voxcpm_amd.engine.lora_manager import LoRABatchPlan, build_lora_batch_plan_from_token_to_slot

    empty = LoRABatchPlan({}, [-1, -1], [], [], [], [0])
    assert (empty.token_indices_sorted_by_slot, empty.active_slot_ids, empty.num_tokens_per_slot, empty.slot_start_offsets) == ([], [], [], [0])
    derived = build_lora_batch_plan_from_token_to_slot({7: 0}, [0, 0, -1, 0])
    assert derived == LoRABatchPlan({7: 0}, [0, 0, -1, 0], [0, 1, 3], [0], [3], [0, 3])
    assert (derived.token_indices_sorted_by_slot, derived.active_slot_ids, derived.num_tokens_per_slot, derived.slot_start_offsets) == ([0, 1, 3], [0], [3], [0, 3])


def test_boundary_rejects_mismatched_tensors_before_any_launch():
    """The ctypes boundary hands raw pointers to the kernels, so what torch's own indexing and
    copy_ would have caught is checked here: element types, devices, lengths, slot range and
    payload shapes (all on host tensors: nothing is launched)."""
    from nanovllm_voxcpm_amd import _hip

    x = torch.zeros(4, 8, dtype=torch.bfloat16)
    y = torch.zeros(4, 16, dtype=torch.bfloat16)
    a, b = torch.zeros(2, 8, 8, dtype=torch.bfloat16), torch.zeros(2, 16, 8, dtype=torch.bfloat16)
    slots = torch.zeros(4, dtype=torch.int32)
    with pytest.raises(ValueError, match="element type"):
        _hip.add_lora(y.float(), x, [a], [b], [0], slots, None, 1.0)
    with pytest.raises(ValueError, match="element type"):
        _hip.add_lora(y, x, [a.half()], [b], [0], slots, None, 1.0)
    with pytest.raises(ValueError, match="3 entries for 4 rows"):
        _hip.add_lora(y, x, [a], [b], [0], slots[:3], None, 1.0)
    with pytest.raises(ValueError, match="int32"):
        _hip.add_lora(y, x, [a], [b], [0], slots.long(), None, 1.0)
    with pytest.raises(ValueError, match="y has 2 rows"):
        _hip.add_lora(y[:2], x, [a], [b], [0], slots, None, 1.0)
    with pytest.raises(RuntimeError, match="no host fallback"):  # everything consistent: only the GPU is missing
        _hip.add_lora(y, x, [a], [b], [0], slots, None, 1.0)
    out = torch.zeros(1, 4, 8, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="token_to_slot"):
        _hip.shrink(x, [a], out, slots[:2], 1.0)
    with pytest.raises(ValueError, match="token_to_slot"):
        _hip.expand(out, [b], y, slots[:1], 0, True)
    with pytest.raises(ValueError, match="element type of y"):
        _hip.expand(out, [b.float()], y, slots, 0, True)
    # slot install
    a_src, b_src = torch.zeros(8, 8), torch.zeros(16, 8)
    with pytest.raises(IndexError, match="outside the 2 slots"):
        _hip.install_slot(a, b, 2, a_src, b_src, 8, 1.0)
    with pytest.raises(ValueError, match="input dim 8"):
        _hip.install_slot(a, b, 0, torch.zeros(8, 4), b_src, 8, 1.0)
    with pytest.raises(ValueError, match="output dim 16"):
        _hip.install_slot(a, b, 0, a_src, torch.zeros(12, 8), 8, 1.0)
    with pytest.raises(ValueError, match="rank 9"):
        _hip.install_slot(a, b, 0, a_src, b_src, 9, 1.0)
    with pytest.raises(ValueError, match="rank 6"):
        _hip.install_slot(a, b, 0, a_src[:4], b_src, 6, 1.0)


def test_layers_refuse_a_slot_outside_their_buffers_before_writing():
    from nanovllm_voxcpm_amd.layers.lora import LoRALinear

    layer = LoRALinear(8, 4, bias=False, max_loras=2, max_lora_rank=4)
    before = layer.lora_A.detach().clone()
    with pytest.raises(IndexError, match="outside the 2 slots"):
        layer.set_slot_lora(2, torch.ones(4, 8), torch.ones(4, 4), effective_rank=4, scaling=1.0)
    with pytest.raises(IndexError, match="outside the 2 slots"):
        layer.clear_slot_lora(-1)
    assert torch.equal(layer.lora_A.detach(), before) and layer._effective_lora_rank_values == [0, 0]


def test_rank_masking_is_requested_only_when_it_can_pay():
    """The layer hands its per-slot rank vector to the backend only for buffers of more than one
    16-rank block that hold an adapter below the padded rank."""
    from nanovllm_voxcpm_amd.layers.lora import LoRALinear

    narrow = LoRALinear(8, 4, bias=False, max_loras=2, max_lora_rank=16)
    narrow.set_slot_lora(0, torch.ones(8, 8), torch.ones(4, 8), effective_rank=8, scaling=1.0)
    assert narrow._wants_rank_masking() is False
    wide = LoRALinear(8, 4, bias=False, max_loras=2, max_lora_rank=64)
    assert wide._wants_rank_masking() is False  # nothing resident
    wide.set_slot_lora(0, torch.ones(64, 8), torch.ones(4, 64), effective_rank=64, scaling=1.0)
    assert wide._wants_rank_masking() is False  # only full-rank adapters
    wide.set_slot_lora(1, torch.ones(8, 8), torch.ones(4, 8), effective_rank=8, scaling=1.0)
    assert wide._wants_rank_masking() is True


def test_rank_masking_under_graph_capture(monkeypatch):
    """A graph captured with nothing resident gets the rank-aware kernels (it must serve what is
    installed later); one captured over full-rank adapters gets the plain ones."""
    from nanovllm_voxcpm_amd.layers import lora as lora_layers

    monkeypatch.setattr(lora_layers, "_is_cuda_graph_capture", lambda: True)
    wide = lora_layers.LoRALinear(8, 4, bias=False, max_loras=2, max_lora_rank=64)
    assert wide._wants_rank_masking() is True
    wide.set_slot_lora(0, torch.ones(64, 8), torch.ones(4, 64), effective_rank=64, scaling=1.0)
    assert wide._wants_rank_masking() is False
    wide.set_slot_lora(1, torch.ones(8, 8), torch.ones(4, 8), effective_rank=8, scaling=1.0)
    assert wide._wants_rank_masking() is True
    narrow = lora_layers.LoRALinear(8, 4, bias=False, max_loras=2, max_lora_rank=16)
    assert narrow._wants_rank_masking() is False


def test_cpp_host_path_loads_and_leaves_what_it_does_not_know_to_python():
    """The C++ host path of the usual add_lora call is built beside the library and loads; it
    registers nothing for tensors that are not on a GPU, and answers "not handled" for weight
    buffers nobody registered, for a missing metadata object and for arguments that are no tensors
    (no compute call is made here: its state object holds no entry points)."""
    import torch

    from nanovllm_voxcpm_amd import _hip

    fc = _hip.load_fastcall()
    assert fc is not None, "make -C nanovllm-voxcpm_amd/csrc fastcall"
    for name in ("create", "register_site", "clear_sites", "set_step", "forget_step", "set_scratch", "counters", "call"):
        assert hasattr(fc, name), name
    state = fc.create(0, 0)
    a, b = [torch.zeros(2, 8, 32)], [torch.zeros(2, 16, 8)]
    x, y = torch.zeros(4, 32), torch.zeros(4, 16)
    slots = torch.zeros(4, dtype=torch.int32)
    args = _hip.MloraAddArgs()
    import ctypes

    assert fc.register_site(state, a, b, (16,), ctypes.addressof(args), args, True) is False  # host tensors
    meta = type("Meta", (), {"no_lora_flag": False, "token_to_slot": slots})()
    assert fc.call(state, [y], x, a, b, slots, meta, 1.0, None, None) == fc.NOT_HANDLED
    assert fc.call(state, [y], x, a, b, slots, None, 1.0, None, None) == fc.NOT_HANDLED
    assert fc.call(state, [y], "x", a, b, slots, meta, 1.0, None, None) == fc.NOT_HANDLED
    assert fc.call(state, [], x, [], [], slots, meta, 1.0, None, None) == fc.NOT_HANDLED
    assert fc.counters(state) == (0, 4)
    fc.clear_sites(state)
    fc.forget_step(state)
