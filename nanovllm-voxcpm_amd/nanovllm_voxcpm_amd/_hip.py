"""ctypes binding of the gfx950 multi-LoRA library (C-ABI declared in include/mlora.h).

The library is built in-tree next to this file.  Nothing here computes: every function
marshals pointers and sizes of torch tensors into the C structs and enqueues HIP work on
torch's current stream.  A missing library is an error, never a silent fallback.
"""

from __future__ import annotations

import contextlib
import ctypes as C
import os
from pathlib import Path

import torch

LIB_NAME = "libmlora_gfx950.so"
LIB_PATH = Path(__file__).resolve().parent / LIB_NAME

MAX_SLICES = 8
MAX_SLOTS = 1024
MAX_RANK = 256

DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
FORM_AUTO, FORM_TOKEN, FORM_BGMV, FORM_SGMV, FORM_MFMA, FORM_SPLIT, FORM_FUSED, FORM_SLOT, FORM_WIDE = 0, 1, 2, 3, 4, 5, 6, 7, 8
FORMS = {"auto": FORM_AUTO, "token": FORM_TOKEN, "bgmv": FORM_BGMV, "sgmv": FORM_SGMV, "mfma": FORM_MFMA, "split": FORM_SPLIT,
         "fused": FORM_FUSED, "slot": FORM_SLOT, "wide": FORM_WIDE}

PLAN_HEADER_WORDS = 16
(
    PLAN_MAGIC,
    PLAN_NUM_TOKENS,
    PLAN_MAX_SLOTS,
    PLAN_NUM_LORA_TOKENS,
    PLAN_NUM_ACTIVE,
    PLAN_NO_LORA,
    PLAN_BAD_SLOT,
    PLAN_TILES_SHORT,
    PLAN_TILES_LONG_SMALL,
    PLAN_TILES_LONG_BIG,
    PLAN_MAX_SEGMENT,
    PLAN_TILES_OVER,
    PLAN_REJECTED,
) = range(13)
PLAN_MAGIC_VALUE = 0x4D4C5031
SEGMENT_THRESHOLD, TILE_SMALL, TILE_BIG = 16, 16, 64
SMALL_TILE_WORDS, SMALL_TILE_ROWS, BIG_TILE_WORDS = 32, 4, 4
STATIC_SCRATCH_BYTES = 16 << 20
WORKSPACE_HEAD_BYTES = 16384 + (4 << 20) + (64 << 10)
WORKSPACE_TIMEOUTS_WORD = 1  # uint32 index in the workspace head: waits of the split form that ran out

_DTYPES = {torch.float32: DTYPE_F32, torch.float16: DTYPE_F16, torch.bfloat16: DTYPE_BF16}

EXPORTS = (
    "mlora_add_lora",
    "mlora_add_lora_static",
    "mlora_add_workspace_bytes",
    "mlora_workspace_init",
    "mlora_shrink",
    "mlora_expand",
    "mlora_plan_workspace_bytes",
    "mlora_meta_build",
    "mlora_install_slot",
    "mlora_stream_capture_id",
    "mlora_abi_version",
    "mlora_last_error",
    "mlora_build_info",
)


# include/mlora_diag.h: measurement and test aids.  The product library exports the first only; the
# diag and trace variants export all three.
DIAG_EXPORTS = ("mlora_reload_knobs", "mlora_probe_launch", "mlora_trace_set")
DIAG_LIB_NAME = "libmlora_gfx950_diag.so"


class MloraSlice(C.Structure):
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("n", C.c_int32), ("y_col", C.c_int32)]


class MloraAddArgs(C.Structure):
    _fields_ = [
        ("stream", C.c_void_p),
        ("x", C.c_void_p),
        ("y", C.c_void_p),
        ("x_stride", C.c_int64),
        ("y_stride", C.c_int64),
        ("token_to_slot", C.c_void_p),
        ("plan", C.c_void_p),
        ("num_tokens", C.c_int32),
        ("k", C.c_int32),
        ("r", C.c_int32),
        ("num_slots", C.c_int32),
        ("num_slices", C.c_int32),
        ("dtype", C.c_int32),
        ("form", C.c_int32),
        ("scaling", C.c_float),
        ("slices", MloraSlice * MAX_SLICES),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_int64),
        ("effective_rank", C.c_void_p),
    ]


class MloraShrinkArgs(C.Structure):
    _fields_ = [
        ("stream", C.c_void_p),
        ("x", C.c_void_p),
        ("out", C.c_void_p),
        ("x_stride", C.c_int64),
        ("token_to_slot", C.c_void_p),
        ("num_tokens", C.c_int32),
        ("k", C.c_int32),
        ("r", C.c_int32),
        ("num_slots", C.c_int32),
        ("num_slices", C.c_int32),
        ("dtype", C.c_int32),
        ("out_dtype", C.c_int32),
        ("scaling", C.c_float),
        ("a", C.c_void_p * MAX_SLICES),
    ]


class MloraExpandArgs(C.Structure):
    _fields_ = [
        ("stream", C.c_void_p),
        ("h", C.c_void_p),
        ("y", C.c_void_p),
        ("y_stride", C.c_int64),
        ("token_to_slot", C.c_void_p),
        ("num_tokens", C.c_int32),
        ("r", C.c_int32),
        ("num_slots", C.c_int32),
        ("num_slices", C.c_int32),
        ("dtype", C.c_int32),
        ("h_dtype", C.c_int32),
        ("offset_start", C.c_int32),
        ("add_inputs", C.c_int32),
        ("b", C.c_void_p * MAX_SLICES),
        ("n", C.c_int32 * MAX_SLICES),
    ]


class MloraMetaArgs(C.Structure):
    _fields_ = [
        ("stream", C.c_void_p),
        ("token_to_slot", C.c_void_p),
        ("num_tokens", C.c_int32),
        ("max_slots", C.c_int32),
        ("no_lora_bucket", C.c_int32),
        ("plan", C.c_void_p),
        ("sorted_idx", C.c_void_p),
        ("compact_ids", C.c_void_p),
        ("compact_counts", C.c_void_p),
        ("compact_offsets", C.c_void_p),
        ("compact_capacity", C.c_int32),
        ("dense_counts", C.c_void_p),
        ("dense_offsets", C.c_void_p),
        ("padded_token_to_slot", C.c_void_p),
        ("padded_len", C.c_int32),
        ("scalars", C.c_void_p),
    ]


class MloraInstallArgs(C.Structure):
    _fields_ = [
        ("stream", C.c_void_p),
        ("a_dst", C.c_void_p),
        ("b_dst", C.c_void_p),
        ("a_src", C.c_void_p),
        ("b_src", C.c_void_p),
        ("a_src_stride", C.c_int64),
        ("b_src_stride", C.c_int64),
        ("slot", C.c_int32),
        ("k", C.c_int32),
        ("n", C.c_int32),
        ("r", C.c_int32),
        ("rank", C.c_int32),
        ("dtype", C.c_int32),
        ("src_dtype", C.c_int32),
        ("scaling", C.c_float),
        ("num_slots", C.c_int32),
    ]


_LIB: C.CDLL | None = None
_LOAD_ERROR: str | None = None


def library_path() -> Path:
    override = os.environ.get("MLORA_LIBRARY")
    return Path(override) if override else LIB_PATH


def load() -> C.CDLL:
    """Load the shared library once; raise RuntimeError with the reason if that fails."""
    global _LIB, _LOAD_ERROR
    if _LIB is not None:
        return _LIB
    if _LOAD_ERROR is not None:
        raise RuntimeError(_LOAD_ERROR)
    path = library_path()
    if not path.exists():
        _LOAD_ERROR = (
            f"HIP multi-LoRA library not built: {path} is missing "
            "(run `make -C nanovllm-voxcpm_amd/csrc` or __graft_entry__.build())"
        )
        raise RuntimeError(_LOAD_ERROR)
    try:
        lib = C.CDLL(str(path))
    except OSError as exc:
        _LOAD_ERROR = f"HIP multi-LoRA library failed to load: {exc}"
        raise RuntimeError(_LOAD_ERROR) from exc
    for name, args in (
        ("mlora_add_lora", MloraAddArgs),
        ("mlora_add_lora_static", MloraAddArgs),
        ("mlora_shrink", MloraShrinkArgs),
        ("mlora_expand", MloraExpandArgs),
        ("mlora_meta_build", MloraMetaArgs),
        ("mlora_install_slot", MloraInstallArgs),
    ):
        fn = getattr(lib, name)
        fn.argtypes = [C.POINTER(args)]
        fn.restype = C.c_int
    lib.mlora_plan_workspace_bytes.argtypes = [C.c_int32, C.c_int32]
    lib.mlora_plan_workspace_bytes.restype = C.c_size_t
    lib.mlora_add_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    lib.mlora_add_workspace_bytes.restype = C.c_size_t
    lib.mlora_workspace_init.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
    lib.mlora_workspace_init.restype = C.c_int
    lib.mlora_stream_capture_id.argtypes = [C.c_void_p]
    lib.mlora_stream_capture_id.restype = C.c_uint64
    _declare_diag(lib)
    lib.mlora_abi_version.argtypes = []
    lib.mlora_abi_version.restype = C.c_int
    lib.mlora_last_error.argtypes = []
    lib.mlora_last_error.restype = C.c_char_p
    lib.mlora_build_info.argtypes = []
    lib.mlora_build_info.restype = C.c_char_p
    _LIB = lib
    return lib


def _declare_diag(lib: C.CDLL) -> None:
    lib.mlora_reload_knobs.argtypes = []
    lib.mlora_reload_knobs.restype = None
    if hasattr(lib, "mlora_probe_launch"):
        lib.mlora_probe_launch.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32]
        lib.mlora_probe_launch.restype = C.c_int
    if hasattr(lib, "mlora_trace_set"):
        lib.mlora_trace_set.argtypes = [C.c_void_p]
        lib.mlora_trace_set.restype = C.c_int


_DIAG_LIB: C.CDLL | None = None


def load_diag() -> C.CDLL:
    """The library that exports the measurement aids of include/mlora_diag.h: the loaded library
    itself when it is a diagnostic variant (MLORA_LIBRARY names the trace build), else the diag
    variant built next to it by `make diag`.  Raises when there is none."""
    global _DIAG_LIB
    if _DIAG_LIB is not None:
        return _DIAG_LIB
    lib = load()
    if not hasattr(lib, "mlora_probe_launch"):
        path = Path(os.environ.get("MLORA_DIAG_LIBRARY") or LIB_PATH.with_name(DIAG_LIB_NAME))
        if not path.exists():
            raise RuntimeError(f"diagnostic variant of the library not built: {path} is missing (run `make -C nanovllm-voxcpm_amd/csrc diag`)")
        lib = C.CDLL(str(path))
        _declare_diag(lib)
        lib.mlora_last_error.argtypes = []
        lib.mlora_last_error.restype = C.c_char_p
    _DIAG_LIB = lib
    return lib


def load_error() -> str | None:
    """Reason the library cannot be used, or None when it loads."""
    try:
        load()
    except RuntimeError as exc:
        return str(exc)
    return None


def load_fastcall():
    """The module with the C++ host path of the usual add_lora call (csrc/fastcall.cpp, built beside
    the library by ``make fastcall``), or None where it is not built or does not load: the Python
    path then does every call.  It launches nothing itself: it calls the library's entry points."""
    try:
        from nanovllm_voxcpm_amd import _mlora_fastcall
    except ImportError:
        return None
    return _mlora_fastcall


def entry_point_addresses() -> tuple[int, int] | None:
    """Addresses of mlora_add_lora and mlora_add_workspace_bytes in the loaded library, None without it."""
    try:
        lib = load()
    except RuntimeError:
        return None
    return C.cast(lib.mlora_add_lora, C.c_void_p).value, C.cast(lib.mlora_add_workspace_bytes, C.c_void_p).value


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().mlora_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"unsupported LoRA element type {dtype}") from None


def _stream(device: torch.device) -> int:
    """Handle of torch's current stream on ``device`` (the raw-handle query is several times
    cheaper than building a ``torch.cuda.Stream`` object, and this runs on every call)."""
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        return raw(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


current_stream_handle = _stream

# torch's own bindings for two questions asked on every call (a foreign call through ctypes costs
# about a microsecond, these a fraction of it); None where this torch build lacks them
_torch_is_capturing = getattr(torch._C, "_cuda_isCurrentStreamCapturing", None)
_torch_get_device = getattr(torch._C, "_cuda_getDevice", None)


def current_device_index() -> int:
    """Index of the calling thread's current GPU."""
    return _torch_get_device() if _torch_get_device is not None else torch.cuda.current_device()


def current_stream_capture_id(device: torch.device, stream: int) -> int:
    """stream_capture_id for ``stream`` = torch's current stream on the calling thread's current
    device ``device``: 0 straight from torch when no capture is in progress there."""
    if _torch_is_capturing is not None and not _torch_is_capturing():
        return 0
    return stream_capture_id(device, stream)

_SAME_DEVICE = contextlib.nullcontext()


def _on(device: torch.device):
    """Context in which ``device`` is the calling thread's current device: a kernel launch goes to
    the current device, whatever stream it names, so a tensor on another GPU of the process has
    to make its device current for the call.  One process per GPU (the reference's deployment)
    never switches."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(device.index)


def _require_cuda(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU; the HIP LoRA path has no host fallback")


def plan_workspace_words(num_tokens: int, max_slots: int) -> int:
    return (load().mlora_plan_workspace_bytes(num_tokens, max_slots) + 3) // 4


_WORKSPACE_BYTES: dict = {}


def add_workspace_bytes(num_tokens: int, num_slices: int, r: int, dtype: torch.dtype) -> int:
    """Bytes of scratch that let the fused apply use every form it has for this shape."""
    key = (num_tokens, num_slices, r, dtype)
    n = _WORKSPACE_BYTES.get(key)
    if n is None:  # asked on every call with the handful of shapes a model has
        if len(_WORKSPACE_BYTES) >= 256:
            _WORKSPACE_BYTES.clear()
        n = _WORKSPACE_BYTES[key] = int(load().mlora_add_workspace_bytes(num_tokens, num_slices, r, dtype_code(dtype)))
    return n


def workspace_init(workspace: torch.Tensor, stream: int | None = None) -> None:
    """Clear the head of a freshly allocated workspace and write its signature (one kernel on
    ``stream``, torch's current one when omitted)."""
    lib = load()
    _require_cuda(workspace, "workspace")
    nbytes = workspace.numel() * workspace.element_size()
    with _on(workspace.device):
        _check(lib.mlora_workspace_init(workspace.data_ptr(), nbytes, _stream(workspace.device) if stream is None else stream),
               "mlora_workspace_init")


def add_lora(
    y: torch.Tensor,
    x: torch.Tensor,
    a_slices: list[torch.Tensor],
    b_slices: list[torch.Tensor],
    y_cols: list[int],
    token_to_slot: torch.Tensor,
    plan: torch.Tensor | None,
    scaling: float,
    form: int = FORM_AUTO,
    workspace: torch.Tensor | None = None,
    stream: int | None = None,
    static_scratch: bool = False,
    effective_rank: torch.Tensor | None = None,
) -> None:
    """y[:, col_i : col_i + n_i] += scaling * (x . A_i[slot]^T) . B_i[slot]^T for every slice.
    ``stream``: handle of the stream to launch on, torch's current one when omitted.
    ``static_scratch``: call the entry point that allocates nothing and keeps its scratch in the
    library's own device image (``workspace`` is ignored then).
    ``effective_rank``: int32 [slots] on the device, rank of the adapter resident in each slot of
    these buffers; rows / columns at or above it are then neither read nor multiplied."""
    lib = load()
    if len(a_slices) > MAX_SLICES:
        raise ValueError(f"at most {MAX_SLICES} slices per call, got {len(a_slices)}")
    dev, dt = x.device, x.dtype  # (names of the offenders are only put together when one is found: this runs per call)
    if token_to_slot.device != dev:
        raise ValueError(f"token_to_slot lives on {token_to_slot.device}, x on {dev}")
    if y.device != dev or y.dtype != dt or any(t.device != dev or t.dtype != dt for t in a_slices) or \
            any(t.device != dev or t.dtype != dt for t in b_slices):
        for name, t in (("y", y), *((f"lora_a[{i}]", a) for i, a in enumerate(a_slices)),
                        *((f"lora_b[{i}]", b) for i, b in enumerate(b_slices))):
            if t.device != dev:
                raise ValueError(f"{name} lives on {t.device}, x on {dev}")
            if t.dtype != dt:
                raise ValueError(f"{name} has element type {t.dtype}, x has {dt}")
    if token_to_slot.dtype != torch.int32 or not token_to_slot.is_contiguous():
        raise ValueError("token_to_slot must be a contiguous int32 tensor")
    if token_to_slot.numel() < x.size(0):
        raise ValueError(f"token_to_slot has {token_to_slot.numel()} entries for {x.size(0)} rows of x")
    if y.size(0) < x.size(0):
        raise ValueError(f"y has {y.size(0)} rows for {x.size(0)} rows of x")
    # the shapes the reference's matmuls would object to (the kernels take K from x and the rank and
    # the slot count from the first A slice: a buffer of another shape would be read with the wrong strides)
    k, r, slots = x.size(1), a_slices[0].size(-2), a_slices[0].size(0)
    for i, (a, b) in enumerate(zip(a_slices, b_slices)):
        if a.dim() != 3 or b.dim() != 3 or a.size(-1) != k or a.size(-2) != r or a.size(0) != slots or b.size(-1) != r or b.size(0) != slots:
            raise ValueError(f"lora_a[{i}] {tuple(a.shape)} / lora_b[{i}] {tuple(b.shape)} do not fit x [{x.size(0)}, {k}] with "
                             f"{slots} slots of rank {r} ([slots, rank, K] and [slots, N, rank] are expected)")
    _require_cuda(x, "x")
    args = MloraAddArgs()
    args.stream = _stream(x.device) if stream is None else stream
    args.x = x.data_ptr()
    args.y = y.data_ptr()
    args.x_stride = x.stride(0)
    args.y_stride = y.stride(0)
    args.token_to_slot = token_to_slot.data_ptr()
    args.plan = plan.data_ptr() if plan is not None else None
    args.num_tokens = x.size(0)
    args.k = x.size(1)
    args.r = a_slices[0].size(-2)
    args.num_slots = a_slices[0].size(0)
    args.num_slices = len(a_slices)
    args.dtype = dtype_code(x.dtype)
    args.form = form
    args.scaling = scaling
    for i, (a, b, col) in enumerate(zip(a_slices, b_slices, y_cols)):
        s = args.slices[i]
        s.a = a.data_ptr()
        s.b = b.data_ptr()
        s.n = b.size(1)
        s.y_col = col
    if workspace is not None:
        args.workspace = workspace.data_ptr()
        args.workspace_bytes = workspace.numel() * workspace.element_size()
    if effective_rank is not None:
        if effective_rank.dtype != torch.int32 or not effective_rank.is_contiguous() or effective_rank.numel() < args.num_slots:
            raise ValueError("effective_rank must be a contiguous int32 tensor with one entry per slot")
        if effective_rank.device != x.device:
            raise ValueError("effective_rank must live on the device of x")
        args.effective_rank = effective_rank.data_ptr()
    with _on(x.device):
        if static_scratch:
            _check(lib.mlora_add_lora_static(C.byref(args)), "mlora_add_lora_static")
        else:
            _check(lib.mlora_add_lora(C.byref(args)), "mlora_add_lora")


def call_add_lora(args: MloraAddArgs) -> None:
    """Enqueue the fused apply described by an argument block the caller filled and checked."""
    rc = load().mlora_add_lora(C.byref(args))
    if rc != 0:
        _check(rc, "mlora_add_lora")


def shrink(
    x: torch.Tensor, a_slices: list[torch.Tensor], out: torch.Tensor, token_to_slot: torch.Tensor, scaling: float
) -> None:
    lib = load()
    if token_to_slot.dtype != torch.int32 or not token_to_slot.is_contiguous() or token_to_slot.numel() < x.size(0):
        raise ValueError(f"token_to_slot must be a contiguous int32 tensor with an entry for each of the {x.size(0)} rows of x")
    for name, t in (("out", out), ("token_to_slot", token_to_slot), *((f"lora_a[{i}]", a) for i, a in enumerate(a_slices))):
        if t.device != x.device:
            raise ValueError(f"{name} lives on {t.device}, x on {x.device}")
    if any(a.dtype != x.dtype for a in a_slices):
        raise ValueError("lora_a slices must have the element type of x")
    if out.size(-2) < x.size(0):
        raise ValueError(f"out has {out.size(-2)} rows for {x.size(0)} rows of x")
    _require_cuda(x, "x")
    args = MloraShrinkArgs()
    args.stream = _stream(x.device)
    args.x = x.data_ptr()
    args.out = out.data_ptr()
    args.x_stride = x.stride(0)
    args.token_to_slot = token_to_slot.data_ptr()
    args.num_tokens = x.size(0)
    args.k = x.size(1)
    args.r = a_slices[0].size(-2)
    args.num_slots = a_slices[0].size(0)
    args.num_slices = len(a_slices)
    args.dtype = dtype_code(x.dtype)
    args.out_dtype = dtype_code(out.dtype)
    args.scaling = scaling
    for i, a in enumerate(a_slices):
        args.a[i] = a.data_ptr()
    with _on(x.device):
        _check(lib.mlora_shrink(C.byref(args)), "mlora_shrink")


def expand(
    h: torch.Tensor,
    b_slices: list[torch.Tensor],
    y: torch.Tensor,
    token_to_slot: torch.Tensor,
    offset_start: int,
    add_inputs: bool,
) -> None:
    lib = load()
    rows = h.size(1)
    if token_to_slot.dtype != torch.int32 or not token_to_slot.is_contiguous() or token_to_slot.numel() < rows:
        raise ValueError(f"token_to_slot must be a contiguous int32 tensor with an entry for each of the {rows} rows")
    for name, t in (("y", y), ("token_to_slot", token_to_slot), *((f"lora_b[{i}]", b) for i, b in enumerate(b_slices))):
        if t.device != h.device:
            raise ValueError(f"{name} lives on {t.device}, the inputs on {h.device}")
    if any(b.dtype != y.dtype for b in b_slices):
        raise ValueError("lora_b slices must have the element type of y")
    if y.size(0) < rows:
        raise ValueError(f"y has {y.size(0)} rows for {rows} rows of the inputs")
    _require_cuda(h, "inputs")
    args = MloraExpandArgs()
    args.stream = _stream(h.device)
    args.h = h.data_ptr()
    args.y = y.data_ptr()
    args.y_stride = y.stride(0)
    args.token_to_slot = token_to_slot.data_ptr()
    args.num_tokens = h.size(1)
    args.r = b_slices[0].size(-1)
    args.num_slots = b_slices[0].size(0)
    args.num_slices = len(b_slices)
    args.dtype = dtype_code(y.dtype)
    args.h_dtype = dtype_code(h.dtype)
    args.offset_start = offset_start
    args.add_inputs = 1 if add_inputs else 0
    for i, b in enumerate(b_slices):
        args.b[i] = b.data_ptr()
        args.n[i] = b.size(1)
    with _on(h.device):
        _check(lib.mlora_expand(C.byref(args)), "mlora_expand")


def _ptr(t: torch.Tensor | None) -> int | None:
    return t.data_ptr() if t is not None else None


def meta_build(
    token_to_slot: torch.Tensor,
    max_slots: int,
    *,
    no_lora_bucket: bool = False,
    plan: torch.Tensor | None = None,
    sorted_idx: torch.Tensor | None = None,
    compact_ids: torch.Tensor | None = None,
    compact_counts: torch.Tensor | None = None,
    compact_offsets: torch.Tensor | None = None,
    compact_capacity: int = 0,
    dense_counts: torch.Tensor | None = None,
    dense_offsets: torch.Tensor | None = None,
    padded_token_to_slot: torch.Tensor | None = None,
    scalars: torch.Tensor | None = None,
) -> None:
    """One launch of the on-device counting sort; every output tensor is optional."""
    lib = load()
    _require_cuda(token_to_slot, "token_to_slot")
    if token_to_slot.dtype != torch.int32 or not token_to_slot.is_contiguous():
        raise ValueError("token_to_slot must be a contiguous int32 tensor")
    args = MloraMetaArgs()
    args.stream = _stream(token_to_slot.device)
    args.token_to_slot = token_to_slot.data_ptr()
    args.num_tokens = token_to_slot.numel()
    args.max_slots = max_slots
    args.no_lora_bucket = 1 if no_lora_bucket else 0
    args.plan = _ptr(plan)
    args.sorted_idx = _ptr(sorted_idx)
    args.compact_ids = _ptr(compact_ids)
    args.compact_counts = _ptr(compact_counts)
    args.compact_offsets = _ptr(compact_offsets)
    args.compact_capacity = compact_capacity
    args.dense_counts = _ptr(dense_counts)
    args.dense_offsets = _ptr(dense_offsets)
    args.padded_token_to_slot = _ptr(padded_token_to_slot)
    args.padded_len = padded_token_to_slot.numel() if padded_token_to_slot is not None else 0
    args.scalars = _ptr(scalars)
    with _on(token_to_slot.device):
        _check(lib.mlora_meta_build(C.byref(args)), "mlora_meta_build")


def install_slot(
    a_dst: torch.Tensor,
    b_dst: torch.Tensor,
    slot: int,
    a_src: torch.Tensor,
    b_src: torch.Tensor,
    rank: int,
    scaling: float,
) -> None:
    """Rewrite one slot of A [slots, r, K] and B [slots, n, r] from an adapter payload."""
    lib = load()
    if not 0 <= slot < a_dst.size(0) or b_dst.size(0) != a_dst.size(0):
        raise IndexError(f"slot {slot} is outside the {a_dst.size(0)} slots of the LoRA buffers")
    if a_src.ndim != 2 or b_src.ndim != 2:
        raise ValueError(f"adapter payload must be 2D, got lora_a {tuple(a_src.shape)} and lora_b {tuple(b_src.shape)}")
    if a_src.size(1) != a_dst.size(2):
        raise ValueError(f"Expected lora_a input dim {a_dst.size(2)}, got {a_src.size(1)}")
    if b_src.size(0) != b_dst.size(1):
        raise ValueError(f"Expected lora_b output dim {b_dst.size(1)}, got {b_src.size(0)}")
    if not 0 <= rank <= a_dst.size(1) or rank > a_src.size(0) or rank > b_src.size(1):
        raise ValueError(f"rank {rank} does not fit the payload {tuple(a_src.shape)} / {tuple(b_src.shape)} and the buffers' rank {a_dst.size(1)}")
    if a_src.stride(1) != 1 or b_src.stride(1) != 1:
        raise ValueError("adapter payload rows must be contiguous")
    if a_src.device != a_dst.device or b_src.device != a_dst.device or b_dst.device != a_dst.device:
        raise ValueError("adapter payload and LoRA buffers must live on one device")
    _require_cuda(a_dst, "lora_A")
    args = MloraInstallArgs()
    args.stream = _stream(a_dst.device)
    args.a_dst = a_dst.data_ptr()
    args.b_dst = b_dst.data_ptr()
    args.a_src = a_src.data_ptr()
    args.b_src = b_src.data_ptr()
    args.a_src_stride = a_src.stride(0)
    args.b_src_stride = b_src.stride(0)
    args.slot = slot
    args.k = a_dst.size(2)
    args.n = b_dst.size(1)
    args.r = a_dst.size(1)
    args.rank = rank
    args.dtype = dtype_code(a_dst.dtype)
    args.src_dtype = dtype_code(a_src.dtype)
    args.scaling = scaling
    args.num_slots = a_dst.size(0)
    with _on(a_dst.device):
        _check(lib.mlora_install_slot(C.byref(args)), "mlora_install_slot")


def stream_capture_id(device: torch.device, stream: int | None = None) -> int:
    """Identifier of the graph capture in progress on ``stream`` (torch's current stream on
    ``device`` when omitted), 0 when none."""
    return int(load().mlora_stream_capture_id(_stream(device) if stream is None else stream))


def reload_knobs() -> None:
    """Make the library read its MLORA_* environment variables again (it keeps them otherwise)."""
    load().mlora_reload_knobs()


def probe_launch(kind: int, buf: torch.Tensor | None = None, grid: tuple[int, int, int] = (1, 1, 1), threads: int = 64,
                 device: torch.device | None = None) -> None:
    """Enqueue a launch of known cost on torch's current stream: kind 0 an empty kernel of the given
    shape, kind 1 a read-modify-write stream over ``buf``, kind 2 a read-only stream over it, kind 3
    a kernel of the given shape whose workgroups each write the XCD they run on into ``buf`` (int32
    per workgroup, linear workgroup order)."""
    dev = buf.device if buf is not None else (device or torch.device("cuda", torch.cuda.current_device()))
    nbytes = buf.numel() * buf.element_size() if buf is not None else 0
    lib = load_diag()
    with _on(dev):
        rc = lib.mlora_probe_launch(_stream(dev), kind, buf.data_ptr() if buf is not None else None, nbytes, *grid, threads)
    if rc != 0:
        raise RuntimeError(f"mlora_probe_launch failed (code {rc}): {lib.mlora_last_error().decode('utf-8', 'replace')}")


def trace_set(buf: torch.Tensor | None) -> None:
    """Hand the trace build of the library a zeroed uint64 [workgroups, 16] buffer to record
    in-kernel timelines into (None switches recording off).  The kernels that record are the
    loaded library's own, so this needs MLORA_LIBRARY to name the trace build; raises otherwise."""
    lib = load()
    if not hasattr(lib, "mlora_trace_set"):
        raise RuntimeError("in-kernel timelines need the trace build of the library (make trace; MLORA_LIBRARY=.../libmlora_gfx950_trace.so)")
    _check(lib.mlora_trace_set(buf.data_ptr() if buf is not None else None), "mlora_trace_set")


def build_info() -> str:
    return load().mlora_build_info().decode()
