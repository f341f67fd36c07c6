"""LoRA backend boundary: the reference's plug point with a HIP backend behind it.

Mirrors the public surface of the reference's ``nanovllm_voxcpm/lora.py``
(``LoRAAvailability``/``LoRAMetadata`` :12-37, the ``LoRABackend`` protocol :40-58,
``get_backend`` / ``set_backend_for_testing`` / ``is_available`` / ``assert_available``
:414-439).  ``HipLoRABackend.add_lora`` replaces ``_VendoredTritonPunicaBackend.add_lora``
(:241-381): one fused launch per call instead of zero + shrink + stack + expand per
(rank, width) bucket, so no slice grouping plan and no pointer tables exist here.

There is no host fallback: without a GPU or without the built library the probed backend is
``_UnavailableBackend`` and every compute method raises.
"""

from __future__ import annotations

import ctypes as C
import os
import struct
import threading
from dataclasses import dataclass
from typing import Protocol

import torch

from nanovllm_voxcpm_amd import _hip
from nanovllm_voxcpm_amd.lora_ops.segment_meta import SegmentPlan, as_slot_vector, build_segment_plan


@dataclass(frozen=True)
class LoRAAvailability:
    available: bool
    reason: str | None = None


@dataclass(frozen=True)
class LoRAMetadata:
    token_to_slot: torch.Tensor | None
    token_indices_sorted_by_slot: torch.Tensor | None
    active_slot_ids: torch.Tensor | None
    num_tokens_per_slot: torch.Tensor | None
    slot_start_offsets: torch.Tensor | None
    no_lora_flag: bool
    num_active_loras: int = 0

    def as_kernel_metadata(self, token_count: int):
        """The 7-tuple the low-level ops take (note: not in field order)."""

        def head(t):
            return None if t is None else t[:token_count]

        return (
            head(self.token_to_slot),
            head(self.token_indices_sorted_by_slot),
            self.num_tokens_per_slot,
            self.slot_start_offsets,
            self.active_slot_ids,
            self.no_lora_flag,
            self.num_active_loras,
        )


class LoRABackend(Protocol):
    def availability(self) -> LoRAAvailability: ...

    def add_lora(
        self,
        y_slices: list[torch.Tensor],
        x: torch.Tensor,
        lora_a_slices: list[torch.Tensor],
        lora_b_slices: list[torch.Tensor],
        *,
        indices: torch.Tensor,
        metadata: LoRAMetadata | None,
        scaling: float,
        y_packed: torch.Tensor | None = None,
    ) -> list[torch.Tensor]: ...

    def shrink(self, x: torch.Tensor, lora_a: torch.Tensor) -> torch.Tensor: ...

    def expand(self, hidden: torch.Tensor, lora_b: torch.Tensor, *, scaling: float) -> torch.Tensor: ...


class _UnavailableBackend:
    """Stands in when the HIP path cannot run; every compute entry raises the reason."""

    def __init__(self, reason: str):
        self.reason = reason

    def availability(self) -> LoRAAvailability:
        return LoRAAvailability(False, self.reason)

    def _refuse(self, *_args, **_kwargs):
        raise RuntimeError(self.reason)

    shrink = expand = add_lora = _refuse


_VECTOR_RANKS = (8, 16, 24, 32, 40, 48, 56, 64)  # rows of B start on 16-byte boundaries and an instance of the kernels covers them
_PLAN_ATTR = "_mlora_segment_plans"
_CONTEXT_PLANS_ATTR = "_mlora_context_plans"  # plan table of the LoRAContext a metadata object was made from


# The per-step fields of MloraAddArgs as they lie in memory: stream, x, y, x_stride, y_stride,
# token_to_slot, plan (eight bytes each, from offset 0) and num_tokens; scaling; workspace,
# workspace_bytes, effective_rank.
_STEP_HEAD = struct.Struct("=QQQqqQQi")
_STEP_SCALE = struct.Struct("=f")
_STEP_TAIL = struct.Struct("=QqQ")
_OFF_SCALING = _hip.MloraAddArgs.scaling.offset
_OFF_WORKSPACE = _hip.MloraAddArgs.workspace.offset
assert _hip.MloraAddArgs.stream.offset == 0 and _hip.MloraAddArgs.num_tokens.offset == 56 and _STEP_HEAD.size == 60
assert _hip.MloraAddArgs.effective_rank.offset == _OFF_WORKSPACE + 16


class _CallSite:
    """What a call of ``add_lora`` derives from its weight tensors alone, kept per set of weight
    buffers (a LoRA linear calls with the same buffers on every step): the filled argument block
    of the C entry point with everything but the per-step fields, and the outcome of the checks
    that concern the weights.  One per thread and set of buffers (addresses, shapes, element type)."""

    __slots__ = ("args", "view", "k", "rank", "num_slots", "dtype", "device", "widths", "weights_vectorisable", "num_slices")


class HipLoRABackend:
    """``LoRABackend`` whose arithmetic runs in the hand-written gfx950 kernels."""

    takes_effective_rank = True  # add_lora accepts the per-slot rank vector of the calling layer

    def __init__(self, form: str | None = None) -> None:
        name = form if form is not None else os.environ.get("MLORA_FORM", "auto")
        if name not in _hip.FORMS:
            raise ValueError(f"unknown LoRA kernel form {name!r}; expected one of {sorted(_hip.FORMS)}")
        self.form = name
        self._scratch: dict = {}
        self._spares: dict = {}          # device -> initialised buffer kept for the next graph capture
        self._graph_scratch: dict = {}   # device -> buffers captured graphs refer to (the last one is in use)
        self._sites = threading.local()  # per thread: weight buffers -> _CallSite
        # the C++ host path of the usual call (optional: built beside the library; MLORA_NO_FASTCALL=1 keeps to Python)
        self._fastcall = None if os.environ.get("MLORA_NO_FASTCALL", "0") not in ("", "0") else _hip.load_fastcall()

    def _fast_state(self):
        """This thread's state object of the C++ host path, None without the module or the library."""
        fc = self._fastcall
        if fc is None:
            return None
        state = getattr(self._sites, "fast", None)
        if state is None:
            addresses = _hip.entry_point_addresses()
            if addresses is None:
                return None
            state = self._sites.fast = fc.create(*addresses)
        return state

    # -- capability ---------------------------------------------------------------------
    def availability(self) -> LoRAAvailability:
        if not torch.cuda.is_available():
            return LoRAAvailability(False, "no ROCm GPU is visible to torch")
        reason = _hip.load_error()
        if reason is not None:
            return LoRAAvailability(False, reason)
        return LoRAAvailability(True, None)

    def prime_slice_caches(
        self,
        lora_a_slices: list[torch.Tensor],
        lora_b_slices: list[torch.Tensor],
        *,
        offset_start: int = 0,
    ) -> None:
        """Nothing to prime: weight pointers travel by value in the launch arguments, so no
        device-side table has to exist before graph capture.  Loading the library here keeps
        the first captured call free of dlopen work."""
        _hip.load()

    # -- segment plan ---------------------------------------------------------------------
    @staticmethod
    def _plan_for(metadata: LoRAMetadata, tts: torch.Tensor, max_slots: int, capture: int | None = None) -> SegmentPlan:
        """One metadata launch per batch: every LoRA layer of a step shares the metadata
        object, so the plan is kept on it.

        Two holders, neither of which can go stale silently:

        * a metadata object made from a ``LoRAContext`` carries the context's own plan table
          (``_mlora_context_plans``).  The plan is then a derived array of the context, like the
          sorted indices and counts the reference keeps there: it lives until the context is
          installed again, is keyed by the slot vector's in-place version where the tensor has
          one, and whoever refreshes the context's buffers in a way the version does not see
          (``graph_meta.copy_lora_domain_to_graph_vars``, inference tensors) drops it;
        * any other metadata object gets a table keyed by the slot vector's address, length and
          in-place version.  Inference tensors have no version counter, so an in-place rewrite
          could not be noticed: for them nothing is kept and every call builds its plan.

        Either way a plan is reused only inside the stream capture it was built in: a plan built
        eagerly during warm-up must not satisfy a later graph capture, or the captured graph
        would contain no metadata launch and replay stale segments.
        """
        own = metadata.token_to_slot
        if own is None or own.data_ptr() != tts.data_ptr():
            return build_segment_plan(tts, max_slots)  # converted / foreign vector: do not cache
        if capture is None:
            capture = _hip.stream_capture_id(tts.device)
        try:
            version = own._version
        except RuntimeError:  # inference tensors carry no version counter
            version = None
        cache = getattr(metadata, _CONTEXT_PLANS_ATTR, None)
        if cache is not None:
            # the version (where the tensor has one) catches an in-place rewrite that nobody
            # announced; writes that bypass the counter are announced by whoever makes them
            key = (tts.data_ptr(), tts.numel(), max_slots, tts.device, version, capture)
        else:
            if version is None:
                return build_segment_plan(tts, max_slots)
            key = (tts.data_ptr(), tts.numel(), max_slots, tts.device, version, capture)
            cache = getattr(metadata, _PLAN_ATTR, None)
            if cache is None:
                cache = {}
                try:
                    object.__setattr__(metadata, _PLAN_ATTR, cache)
                except (AttributeError, TypeError):
                    return build_segment_plan(tts, max_slots)  # slotted metadata type
        plan = cache.get(key)
        if plan is None:
            if len(cache) >= 4:
                cache.clear()
            plan = cache[key] = build_segment_plan(tts, max_slots)
        return plan

    def _new_scratch(self, device: torch.device, nbytes: int, stream: int | None) -> torch.Tensor:
        buf = torch.empty(max(nbytes, 4 << 20), dtype=torch.uint8, device=device)
        _hip.workspace_init(buf, stream)  # one kernel, once per buffer: head cleared, signature written
        return buf

    def _scratch_for(self, x: torch.Tensor, num_slices: int, rank: int, stream: int | None = None,
                     capture: int | None = None) -> torch.Tensor:
        """Device scratch for the rank-r intermediate (between the two launches of the
        long-segment form, or between producer and consumer workgroups of the split form).

        Eager calls: one buffer per (device, stream), grown on demand - calls on one stream are
        ordered, so they can share it.  When the table is full its oldest entry goes, not all.

        Graphs being captured: one buffer per device, shared by every graph this backend captures
        there and always allocated and initialised OUTSIDE the capture (every eager call keeps
        one ready), so that no graph holds an initialisation launch or memory of its own for it.
        The graphs refer to it for as long as they live, so it is only ever replaced by a larger
        one (the smaller stays alive with them).  Sharing is safe under the rule that holds for
        every workspace - launches that use it are ordered on one stream: the engine replays its
        graphs one after the other on one stream.  Without a buffer ready (a capture as the very
        first call, or one that needs more than any eager call did) the buffer comes from the
        graph's own pool and its initialisation is recorded with it."""
        nbytes = _hip.add_workspace_bytes(x.size(0), num_slices, rank, x.dtype)
        if stream is None:
            stream = _hip.current_stream_handle(x.device)
        if capture is None:
            capture = _hip.stream_capture_id(x.device, stream)
        device = x.device
        if capture:
            held = self._graph_scratch.get(device)
            if held is not None and held[-1].numel() >= nbytes:
                return held[-1]
            spare = self._spares.pop(device, None)
            if spare is not None and spare.numel() >= nbytes:
                self._graph_scratch.setdefault(device, []).append(spare)
                return spare
            if spare is not None:
                self._spares[device] = spare
            key = (device, stream, capture)  # from the graph's own pool, initialisation recorded
            buf = self._scratch.get(key)
            if buf is None or buf.numel() < nbytes:
                buf = self._scratch[key] = self._new_scratch(device, nbytes, stream)
            return buf
        key = (device, stream, 0)
        buf = self._scratch.get(key)
        if buf is None or buf.numel() < nbytes:
            if buf is None and len(self._scratch) >= 8:
                del self._scratch[next(iter(self._scratch))]  # the oldest entry (its stream's work is queued behind it)
            buf = self._scratch[key] = self._new_scratch(device, nbytes, stream)
        # a buffer for the next capture, as large as the largest eager one: made here, outside any capture
        need = buf.numel()
        held = self._graph_scratch.get(device)
        if (held is None or held[-1].numel() < need) and (device not in self._spares or self._spares[device].numel() < need):
            self._spares[device] = self._new_scratch(device, need, stream)
        return buf

    def scratch_buffers(self) -> list[torch.Tensor]:
        """Every scratch buffer this backend holds (eager ones and those captured graphs refer to)."""
        return list(self._scratch.values()) + [buf for held in self._graph_scratch.values() for buf in held] + list(self._spares.values())

    @staticmethod
    def _vectorisable(x: torch.Tensor, y: torch.Tensor, a_list, b_list, cols) -> bool:
        """Host mirror of the library's test for the 128-bit kernels (a plan is only built when
        it can be used)."""
        if x.dtype not in (torch.float16, torch.bfloat16):
            return False
        if a_list[0].size(-2) not in _VECTOR_RANKS:
            return False
        if x.size(1) % 8 or x.stride(0) % 8 or y.stride(0) % 8 or x.data_ptr() % 16 or y.data_ptr() % 16:
            return False
        for a, b, col in zip(a_list, b_list, cols):
            if b.size(1) % 8 or col % 8 or a.data_ptr() % 16 or b.data_ptr() % 16:
                return False
        return True

    # -- the usual call, with what the weights determine kept per set of buffers -----------------
    def _site_for(self, a_list, b_list, widths) -> "_CallSite | None":
        """The call site of these weight buffers, made on first use; None when the call is not of
        the usual kind (slices of different rank or K, an empty slice, too many slices), which the
        general path below then handles."""
        key = []
        for t in a_list:
            key.append(t.data_ptr())
            key.append(t.shape)
        for t in b_list:
            key.append(t.data_ptr())
            key.append(t.shape)
        a0 = a_list[0]
        key.append(a0.dtype)
        key = tuple(key)
        table = getattr(self._sites, "table", None)
        if table is None:
            table = self._sites.table = {}
        site = table.get(key)
        if site is not None:
            return site if site.widths == widths else None
        if len(a_list) > _hip.MAX_SLICES or a0.dim() != 3 or any(w == 0 for w in widths):
            return None
        rank, k, slots = a0.size(-2), a0.size(-1), a0.size(0)
        dev, dt = a0.device, a0.dtype
        for a, b, w in zip(a_list, b_list, widths):
            if a.dim() != 3 or b.dim() != 3 or a.size(-2) != rank or a.size(-1) != k or a.size(0) != slots or b.size(0) != slots:
                return None
            if b.size(-1) != rank or b.size(1) != w or a.device != dev or b.device != dev or a.dtype != dt or b.dtype != dt:
                return None
        if not a0.is_cuda or dt not in _hip._DTYPES:
            return None
        site = _CallSite()
        args = site.args = _hip.MloraAddArgs()
        args.k, args.r, args.num_slots, args.num_slices, args.dtype = k, rank, slots, len(a_list), _hip.dtype_code(dt)
        args.form = _hip.FORMS[self.form]
        col, ok = 0, dt in (torch.float16, torch.bfloat16) and rank in _VECTOR_RANKS and k % 8 == 0
        for i, (a, b, w) in enumerate(zip(a_list, b_list, widths)):
            sl = args.slices[i]
            sl.a, sl.b, sl.n, sl.y_col = a.data_ptr(), b.data_ptr(), w, col
            ok = ok and w % 8 == 0 and col % 8 == 0 and a.data_ptr() % 16 == 0 and b.data_ptr() % 16 == 0
            col += w
        # (no reference to the tensors is kept: the key is their addresses, shapes and element type,
        # so whatever answers to the key later lies where the block says)
        site.view = memoryview(args).cast("B")
        site.k, site.rank, site.num_slots, site.dtype, site.device, site.widths = k, rank, slots, dt, dev, widths
        site.weights_vectorisable, site.num_slices = ok, len(a_list)
        fast = self._fast_state()
        if len(table) >= 512:
            table.clear()
            if fast is not None:
                self._fastcall.clear_sites(fast)
        table[key] = site
        if fast is not None:  # (it keeps the block alive itself; its key is the one above)
            self._fastcall.register_site(fast, a_list, b_list, widths, C.addressof(args), args, ok)
        return site

    def _add_lora_at_site(self, outputs, target, x, a_list, b_list, indices, metadata, scaling, effective_rank) -> bool:
        """The usual call - every slice non-empty, all of one rank and K, unit column strides - with
        the argument block of its weight buffers reused from the last step: only what changes per
        step (activations, slot vector, plan, scratch, stream) is entered.  Returns False, having
        done nothing, for anything else and for everything that has to raise: the general path
        then runs, with its checks and their messages."""
        if x.dim() != 2 or x.stride(1) != 1 or target.dim() != 2 or target.stride(1) != 1:
            return False
        widths = tuple([y.size(-1) for y in outputs])
        site = self._site_for(a_list, b_list, widths)
        if site is None:
            return False
        rows = x.size(0)
        source = metadata.token_to_slot if metadata.token_to_slot is not None else indices
        if (x.size(1) != site.k or x.dtype != site.dtype or target.dtype != site.dtype or x.device != site.device or
                target.device != site.device or source.device != site.device or source.numel() < rows or target.size(0) < rows or
                source.dtype != torch.int32 or not source.is_contiguous() or source.dim() != 1):
            return False
        x_ptr, y_ptr, xs, ys = x.data_ptr(), target.data_ptr(), x.stride(0), target.stride(0)
        args = site.args
        eff_ptr = 0
        if effective_rank is not None:
            if (effective_rank.dtype != torch.int32 or not effective_rank.is_contiguous() or effective_rank.numel() < site.num_slots or
                    effective_rank.device != site.device):
                return False
            eff_ptr = effective_rank.data_ptr()
        dev = site.device
        if dev.index is not None and dev.index != _hip.current_device_index():
            return False  # another GPU of this process: the general path makes it current
        stream = _hip.current_stream_handle(dev)
        plan_ptr = ws_ptr = ws_bytes = 0
        if site.weights_vectorisable and args.form != _hip.FORM_TOKEN and not (xs % 8 or ys % 8 or x_ptr % 16 or y_ptr % 16):
            capture = _hip.current_stream_capture_id(dev, stream)
            # every LoRA linear of a step calls with the same metadata object, slot vector, stream
            # and capture: what the last call of this thread looked up serves the next one
            try:
                version = source._version
            except RuntimeError:  # inference tensors carry no version counter: nothing is remembered for them
                version = None
            memo = getattr(self._sites, "step", None)
            if (memo is not None and version is not None and memo[0] is metadata and memo[1] is source and memo[2] == version and
                    memo[3] == capture and memo[4] == stream and memo[5] == site.num_slots and memo[6] == rows):
                plan_ptr = memo[7]
            else:
                tts = source if source.numel() == rows else source[:rows]
                plan = self._plan_for(metadata, tts, site.num_slots, capture)
                plan_ptr = plan.workspace.data_ptr()
                # (the plan object is part of the memo: its workspace stays allocated while it is remembered)
                self._sites.step = (metadata, source, version, capture, stream, site.num_slots, rows, plan_ptr, plan)
                fast = self._fast_state()
                if fast is not None:
                    if capture or version is None:
                        self._fastcall.forget_step(fast)
                    else:  # (the tuple above keeps metadata, slot vector and plan alive for as long as this stands)
                        self._fastcall.set_step(fast, metadata, source, version, stream or 0, site.num_slots, rows, plan_ptr)
            scratch = self._scratch_for(x, site.num_slices, site.rank, stream, capture)
            ws_ptr, ws_bytes = scratch.data_ptr(), scratch.numel()
            if not capture:
                fast = self._fast_state()
                if fast is not None:  # (held in self._scratch for as long as it is the stream's buffer)
                    self._fastcall.set_scratch(fast, dev.index if dev.index is not None else _hip.current_device_index(), stream or 0, ws_ptr, ws_bytes)
        # the per-step fields, written in three strokes (they lie together in the block; one attribute
        # assignment per field costs several times as much)
        _STEP_HEAD.pack_into(site.view, 0, stream or 0, x_ptr, y_ptr, xs, ys, source.data_ptr(), plan_ptr, rows)
        _STEP_SCALE.pack_into(site.view, _OFF_SCALING, scaling)
        _STEP_TAIL.pack_into(site.view, _OFF_WORKSPACE, ws_ptr, ws_bytes, eff_ptr)
        _hip.call_add_lora(args)
        return True

    # -- the fused apply -------------------------------------------------------------------
    def add_lora(
        self,
        y_slices: list[torch.Tensor],
        x: torch.Tensor,
        lora_a_slices: list[torch.Tensor],
        lora_b_slices: list[torch.Tensor],
        *,
        indices: torch.Tensor,
        metadata: LoRAMetadata | None,
        scaling: float,
        y_packed: torch.Tensor | None = None,
        effective_rank: torch.Tensor | None = None,
    ) -> list[torch.Tensor]:
        """y_i[t] += scaling * (x[t] . A_i[slot_t]^T) . B_i[slot_t]^T for every slice i and every
        token with a slot; rows with slot -1 keep their bits.

        ``effective_rank`` (beyond the reference's protocol, optional): int32 [slots] on the
        device, the rank of the adapter resident in each slot of these buffers
        (``layer.effective_lora_rank``).  Rows of A and columns of B at or above it are then
        neither read nor multiplied.

        With ``y_packed`` the slices must be its column blocks in order (``split`` views) and
        are updated in place; a single slice is updated in place; several slices without
        ``y_packed`` are gathered into a new packed buffer whose views are returned and the
        caller's tensors stay untouched (reference: nanovllm_voxcpm/lora.py:276-289).
        """
        fast = getattr(self._sites, "fast", None)
        if fast is not None:
            # the usual call, when nothing about it is new: checked, filled in and enqueued in C++
            rc = self._fastcall.call(fast, y_slices, x, lora_a_slices, lora_b_slices, indices, metadata, scaling, y_packed, effective_rank)
            if rc == 0:
                return list(y_slices)
            if rc < 0:
                _hip._check(rc, "mlora_add_lora")
        if not y_slices:
            return []
        if not (len(y_slices) == len(lora_a_slices) == len(lora_b_slices)):
            raise ValueError("add_lora expects aligned y/lora_a/lora_b slice lists")
        if metadata is None:
            raise RuntimeError("LoRA metadata must be prepared by the model runner before backend execution")
        for a in lora_a_slices:
            if not a.is_contiguous():
                raise ValueError("add_lora expects contiguous lora_a slices")
        for b in lora_b_slices:
            if not b.is_contiguous():
                raise ValueError("add_lora expects contiguous lora_b slices")

        outputs = list(y_slices)
        if y_packed is not None:
            if y_packed.dim() != 2:
                raise ValueError("y_packed must be 2D [num_tokens, packed_hidden]")
            target = y_packed
        elif len(y_slices) == 1:
            target = y_slices[0]
        else:
            widths = [y.size(-1) for y in y_slices]
            target = torch.cat(y_slices, dim=-1)
            outputs = list(target.split(widths, dim=-1))

        if metadata.no_lora_flag or x.size(0) == 0:
            return outputs

        if self._add_lora_at_site(outputs, target, x, lora_a_slices, lora_b_slices, indices, metadata, scaling, effective_rank):
            return outputs

        cols, col = [], 0
        for i, y in enumerate(outputs):
            cols.append(col)
            col += y.size(-1)
            if y.numel() > 0 and lora_b_slices[i].dim() == 3 and lora_b_slices[i].size(1) != y.size(-1):  # (empty slices are skipped)
                raise ValueError(f"y slice {i} has {y.size(-1)} columns, lora_b[{i}] {tuple(lora_b_slices[i].shape)} gives {lora_b_slices[i].size(1)}")
        live = [i for i, y in enumerate(outputs) if y.numel() > 0]
        if not live:
            return outputs

        source = metadata.token_to_slot if metadata.token_to_slot is not None else indices
        if source.numel() < x.size(0):
            raise ValueError(f"LoRA slot vector has {source.numel()} entries for {x.size(0)} rows of x")
        tts = as_slot_vector(source[: x.size(0)])
        if not tts.is_cuda:
            raise RuntimeError("LoRA slot ids must live on the GPU; the HIP LoRA path has no host fallback")
        if target.size(0) < x.size(0):
            raise ValueError(f"y has {target.size(0)} rows for {x.size(0)} rows of x")

        x2 = x if x.stride(-1) == 1 else x.contiguous()
        staged = None
        if target.stride(-1) != 1:
            staged, target = target, target.contiguous()

        # Slices are launched together when they share (rank, K); shapes that differ (never
        # the case for the stacked projections) simply take one launch each.
        stream = _hip.current_stream_handle(x2.device)  # looked up once per call
        capture = None
        groups: dict[tuple[int, int], list[int]] = {}
        for i in live:
            a = lora_a_slices[i]
            groups.setdefault((a.size(-2), a.size(-1)), []).append(i)
        for members in groups.values():
            for lo in range(0, len(members), _hip.MAX_SLICES):
                chunk = members[lo : lo + _hip.MAX_SLICES]
                a_list = [lora_a_slices[i] for i in chunk]
                b_list = [lora_b_slices[i] for i in chunk]
                c_list = [cols[i] for i in chunk]
                plan = scratch = None
                form = _hip.FORMS[self.form]
                if form != _hip.FORM_TOKEN and self._vectorisable(x2, target, a_list, b_list, c_list):
                    if capture is None:
                        capture = _hip.stream_capture_id(x2.device, stream)
                    plan = self._plan_for(metadata, tts, a_list[0].size(0), capture).workspace
                    scratch = self._scratch_for(x2, len(chunk), a_list[0].size(-2), stream, capture)
                _hip.add_lora(target, x2, a_list, b_list, c_list, tts, plan, float(scaling), form, scratch, stream,
                              effective_rank=effective_rank)
        if staged is not None:
            staged.copy_(target)
        return outputs

    # -- single-adapter helpers of the protocol -----------------------------------------------
    def shrink(self, x: torch.Tensor, lora_a: torch.Tensor) -> torch.Tensor:
        """x . lora_a^T for one adapter ([rank, K] or [1, rank, K]); result in x's dtype."""
        a = lora_a.unsqueeze(0) if lora_a.ndim == 2 else lora_a
        a = a.contiguous()
        x2 = x if x.stride(-1) == 1 else x.contiguous()
        out = torch.empty((1, x.size(0), a.size(-2)), dtype=x.dtype, device=x.device)
        slots = torch.zeros(x.size(0), dtype=torch.int32, device=x.device)
        _hip.shrink(x2, [a], out, slots, 1.0)
        return out.squeeze(0)

    def expand(self, hidden: torch.Tensor, lora_b: torch.Tensor, *, scaling: float) -> torch.Tensor:
        """(hidden . lora_b^T) * scaling for one adapter ([N, rank] or [1, N, rank])."""
        b = lora_b.unsqueeze(0) if lora_b.ndim == 2 else lora_b
        b = b.contiguous()
        out = torch.zeros(hidden.size(0), b.size(1), dtype=hidden.dtype, device=hidden.device)
        slots = torch.zeros(hidden.size(0), dtype=torch.int32, device=hidden.device)
        _hip.expand(hidden.contiguous().unsqueeze(0), [b], out, slots, 0, False)
        return out * scaling


_BACKEND_OVERRIDE: LoRABackend | None = None
_PROBED_BACKEND: LoRABackend | None = None


def _probe_backend() -> LoRABackend:
    backend = HipLoRABackend()
    status = backend.availability()
    if status.available:
        return backend
    return _UnavailableBackend(status.reason or "HIP multi-LoRA kernels are unavailable")


def get_backend() -> LoRABackend:
    global _PROBED_BACKEND
    if _BACKEND_OVERRIDE is not None:
        return _BACKEND_OVERRIDE
    if _PROBED_BACKEND is None:
        _PROBED_BACKEND = _probe_backend()
    return _PROBED_BACKEND


def set_backend_for_testing(backend: LoRABackend | None) -> None:
    global _BACKEND_OVERRIDE
    _BACKEND_OVERRIDE = backend


def get_availability() -> LoRAAvailability:
    return get_backend().availability()


def is_available() -> bool:
    return get_availability().available


def assert_available() -> None:
    status = get_availability()
    if not status.available:
        raise RuntimeError(status.reason or "LoRA runtime is unavailable")
