// Entry points declared in include/mlora.h.  mlora_add_lora stands where the reference's backend
// method stands (nanovllm_voxcpm/lora.py:241-381); its slice grouping plan (lora.py:65-90, 195-239)
// and pointer tables (lora_ops/triton_ops/utils.py:15-116) have no counterpart: one launch takes a
// table of slices with their own widths, and pointers travel by value.
//
// C-ABI front door: argument checks, form selection, error text.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include <mutex>

#include "common.h"
#include "launch.h"
#include "mlora_diag.h"

namespace mlora {

namespace {
thread_local char g_error[512] = "";
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return static_cast<int>(e);
  }
  return 0;
}

namespace {
int g_knob_generation = 0;
}
int knob_generation() { return g_knob_generation; }

int env_int(const char* name, int fallback) {
  const char* v = getenv(name);
  if (!v || !*v) return fallback;
  return atoi(v);
}

}  // namespace mlora

using namespace mlora;

namespace {

// Both matrix-core forms step through K in units of 32.
bool mfma_supported(const MloraAddArgs* a) { return a->k % 32 == 0 && a->k >= 32; }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// The vectorised kernels move eight 16-bit elements per lane: every row they touch has to
// start on a 16-byte boundary.
bool vector_ok(const MloraAddArgs* a) {
  if (a->dtype != MLORA_DTYPE_F16 && a->dtype != MLORA_DTYPE_BF16) return false;
  if (!a->plan) return false;
  if (!padded_rank(a->r)) return false;  // 8, 16, 24, ... 64: rows of B start on 16-byte boundaries
  if (a->k % 8 || a->x_stride % 8 || a->y_stride % 8) return false;
  if (!aligned16(a->x) || !aligned16(a->y)) return false;
  for (int i = 0; i < a->num_slices; ++i) {
    const MloraSlice& s = a->slices[i];
    if (s.n % 8 || s.y_col % 8 || !aligned16(s.a) || !aligned16(s.b)) return false;
  }
  return true;
}

}  // namespace

namespace {

// Diagnostic knobs, read from the environment once per process.
struct ApiKnobs {
  int generation = -1, small_batch_tokens, force_form, no_split, split_min_rk, split_max_tokens, auto_fused, slot_max_slots, no_wide;
  void read() {
    generation = knob_generation();
    small_batch_tokens = env_int("MLORA_SMALL_BATCH_TOKENS", 0);
    force_form = env_int("MLORA_FORCE_FORM", 0);
    no_split = env_int("MLORA_NO_SPLIT", 0);
    // Measured on the prefill batch (7605 tokens, rank 64) and the mixed one: the one-launch
    // long-segment form takes 4060 us per step against 3586 for two launches (mixed: 6090 against
    // 4992).  Its workgroups are all resident at once, so the whole grid first shrinks (a chain of
    // dependent slab fetches per workgroup, HBM nearly idle) and then expands; the saved launch
    // does not pay for the wait on the slowest role of each unit.  AUTO keeps the two launches.
    auto_fused = env_int("MLORA_AUTO_FUSED", 0);
    no_wide = env_int("MLORA_NO_WIDE", 0);
    // The split form pays when A[slot], which every workgroup of a tile would otherwise fetch whole,
    // is large: rank x K >= 131072 elements (256 KB).  Measured on the decode batch (256 tokens, 32
    // adapters), one workgroup per (tile, column range) against the split form, us per call: rank 16,
    // K = 4096: 6.9 / 8.0 (what producers publish reaches the consumers 1.6 us later, two trips
    // through the memory system; more than spreading 128 KB saves); rank 32, K = 4096: 15.5 / 10.5;
    // rank 32, K = 1024: 4.9-10.0 / 8.1-17.1; rank 16, K = 8192: the K range of a workgroup no
    // longer fits its registers as one batch of loads.
    split_min_rk = env_int("MLORA_SPLIT_MIN_RK", 131072);
    // ... and while the batch has few tiles: K = 4096, rank 32 / 64, 1011 tokens: 12.0 / 17.7 us against
    // 14.8 / 23.1; 1620 tokens: 17.6 / 26.8 against 15.8 / 24.7
    split_max_tokens = env_int("MLORA_SPLIT_MAX_TOKENS", 1280);
    // The slot-major grid launches a workgroup per (slot id, column range) whether the slot has
    // tokens or not; with many more slot ids than adapters in the batch those requests are waste.
    slot_max_slots = env_int("MLORA_SLOT_MAX_SLOTS", 64);
  }
};
const ApiKnobs& knobs() {
  static ApiKnobs k;
  if (k.generation != knob_generation()) k.read();
  return k;
}

}  // namespace

// Where the one-launch form over 16-token tiles stops paying.  Its cost per token grows with the
// rank (every tile fetches A[slot] and B[slot] again, every column range repeats its tile's shrink)
// while a two-launch call pays about 10 us before it moves any data (3.5 us for one launch over
// small tiles).  Measured per projection shape on prefill batches of 1011..9392 tokens (1..16
// sequences, up to 8 adapters), the two forms meet where tokens x width reaches about 1.5e7-1.7e7
// at rank 64, 2.6e7 at rank 32 and 8.3e7 at rank 16, with width = slices x K x max(1, K / 1024) +
// columns x max(1, columns / 4096): long K and wide outputs cost the small tiles more than their
// share (tokens at the crossing, rank 64 / 32 / 16: qkv 4000 / 6000 / 19000, o 8300 / 12700 / -,
// gate_up 900 / 1400 / 4500, down 1000 / 1500 / 4800).
// The rank-64 limit is 1.5e7: with many adapters in the batch the small tiles lose earlier (the
// mixed batch, 8192 tokens and 128 adapters: o 28.8 us per call on small tiles, 23.0 in two launches).
// Where the other form would be the one-launch form over 64-token tiles (`one_launch`), which
// pays about half as much before it moves data, the small tiles lose earlier: measured on the same
// batches, us per call over small tiles / in one launch over 64-token tiles, by tokens of the batch:
// rank 64, qkv: 14.8 / 14.3 at 1620, 15.4 / 14.6 at 2098, 18.0 / 15.0 at 3250, 21.2 / 15.5 at 4511;
// o: 10.5 / 14.8 at 4511, 18.1 / 15.2 at 6648; rank 32, qkv: 11.5 / 12.3 at 3250, 14.4 / 12.8 at 4511;
// o: 12.4 / 12.6 at 6648, 13.9 / 14.8 at 9392: the limits are 0.65 times the above there.
// MLORA_SMALL_BATCH_TOKENS, when set, replaces the rule by a plain token count.
static bool small_batch(const MloraAddArgs* a, bool one_launch) {
  const int fixed = knobs().small_batch_tokens;
  if (fixed > 0) return a->num_tokens <= fixed;
  double cols = 0;
  for (int i = 0; i < a->num_slices; ++i) cols += a->slices[i].n;
  const double width = static_cast<double>(a->num_slices) * a->k * (a->k > 1024 ? a->k / 1024.0 : 1.0) + cols * (cols > 4096 ? cols / 4096.0 : 1.0);
  const double limit = (a->r <= 16 ? 8.3e7 : a->r <= 32 ? 2.6e7 : 1.5e7) * (one_launch ? 0.65 : 1.0);
  return a->num_tokens * width <= limit;
}

// Where the slot-major grid pays.  Its workgroups request the weights of EVERY slot id, with or
// without tokens, so what it costs grows with the slot ids nobody uses: measured on decode batches of
// 4..256 tokens over 32 slot ids (us per call, slot-major / tile-major): gate_up, whose slots weigh
// 327 KB each, 5.9 / 3.9 at 4 tokens, 5.6 / 5.2 at 64, 6.1 / 6.0 at 128, 6.7 / 6.8 at 256; o (64 KB per
// slot) 3.5 / 3.4 at 4 tokens, 3.7 / 3.8 at 64, 3.8 / 4.1 at 256; over 8 slot ids it is the faster
// grid at every batch size and every projection; with 128 slot ids of which 32 are in use it
// takes 967 us per decode step against 629.  With K shared out between a tile's workgroups (down) it
// is the faster one throughout (5.2 / 5.6 at 4 tokens, 6.4 / 6.8 at 256).  So: always with K parts;
// else while all slots together weigh at most 3 MB, or when the batch has four tokens per slot id.
// All of this was measured on decode batches; on batches of many tiles per slot (a prefill of
// 2098 tokens over 8 slot ids, o: 15.4 us per call against 10.1 tile-major) the grid over the slots
// is the slower one: it is taken up to 32 tokens per slot id.
static bool slot_major_pays(const MloraAddArgs* a) {
  if (a->num_slots > knobs().slot_max_slots) return false;
  if (a->num_tokens > 32 * a->num_slots) return false;
  if (slot_k_parts(a) > 1) return true;
  double cols = 0;
  for (int i = 0; i < a->num_slices; ++i) cols += a->slices[i].n;
  const double per_slot = 2.0 * a->r * (static_cast<double>(a->num_slices) * a->k + cols);
  if (a->num_slots * per_slot <= 3.0e6) return true;
  return a->num_tokens >= 4 * a->num_slots;
}

namespace {

int add_lora_impl(const MloraAddArgs* a, bool trusted_workspace);

}  // namespace

extern "C" int mlora_add_lora(const MloraAddArgs* a) { return add_lora_impl(a, false); }

namespace {

int add_lora_impl(const MloraAddArgs* a, bool trusted_workspace) {
  if (!a) { set_error("mlora_add_lora: NULL args"); return MLORA_E_INVALID; }
  if (a->num_tokens < 0 || a->k < 0 || a->r < 0 || a->num_slots < 0 || a->num_slices < 0) {
    set_error("mlora_add_lora: negative size"); return MLORA_E_INVALID;
  }
  if (a->dtype != MLORA_DTYPE_F32 && a->dtype != MLORA_DTYPE_F16 && a->dtype != MLORA_DTYPE_BF16) {
    set_error("mlora_add_lora: unknown dtype %d", a->dtype); return MLORA_E_INVALID;
  }
  if (a->form < MLORA_FORM_AUTO || a->form > MLORA_FORM_WIDE) { set_error("mlora_add_lora: unknown form %d", a->form); return MLORA_E_INVALID; }
  if (a->num_slices > MLORA_MAX_SLICES) { set_error("mlora_add_lora: %d slices exceed %d", a->num_slices, MLORA_MAX_SLICES); return MLORA_E_TOO_LARGE; }
  if (a->r > MLORA_MAX_RANK) { set_error("mlora_add_lora: rank %d exceeds %d", a->r, MLORA_MAX_RANK); return MLORA_E_TOO_LARGE; }
  if (a->num_slots > MLORA_MAX_SLOTS) { set_error("mlora_add_lora: %d slots exceed %d", a->num_slots, MLORA_MAX_SLOTS); return MLORA_E_TOO_LARGE; }
  if (a->num_tokens == 0 || a->num_slices == 0 || a->num_slots == 0 || a->r == 0) return 0;
  if (!a->x || !a->y || !a->token_to_slot) { set_error("mlora_add_lora: NULL tensor pointer"); return MLORA_E_INVALID; }
  bool any = false;
  for (int i = 0; i < a->num_slices; ++i) {
    const MloraSlice& s = a->slices[i];
    if (s.n < 0 || s.y_col < 0) { set_error("mlora_add_lora: slice %d has negative extent", i); return MLORA_E_INVALID; }
    if (s.n > 0 && (!s.a || !s.b)) { set_error("mlora_add_lora: slice %d has NULL weights", i); return MLORA_E_INVALID; }
    if (static_cast<int64_t>(s.y_col) + s.n > a->y_stride) {
      set_error("mlora_add_lora: slice %d ends at column %lld, beyond the y row stride %lld", i, static_cast<long long>(s.y_col) + s.n,
                static_cast<long long>(a->y_stride));
      return MLORA_E_INVALID;
    }
    any |= s.n > 0;
  }
  if (a->x_stride < a->k) { set_error("mlora_add_lora: x row stride %lld is below K = %d", static_cast<long long>(a->x_stride), a->k); return MLORA_E_INVALID; }
  if (!any) return 0;
  if (reinterpret_cast<uintptr_t>(a->plan) & 15) { set_error("mlora_add_lora: plan must be 16-byte aligned"); return MLORA_E_INVALID; }

  int form = a->form;
  const bool vec = vector_ok(a);
  if (form == MLORA_FORM_AUTO) {
    const int forced = knobs().force_form;
    if (forced >= MLORA_FORM_TOKEN && forced <= MLORA_FORM_WIDE && (forced == MLORA_FORM_TOKEN || vec)) form = forced;
  }
  if (form == MLORA_FORM_AUTO) {
    // Small batches (decode) are one launch over 16-token tiles; large ones split into 64-token
    // tiles for the long segments and 16-token tiles for the rest: one launch whose workgroups do
    // both products where a tile's column ranges repeat little of its shrink, else two launches.
    const bool small_tiles = mfma_supported(a) && decode_supported(a);
    const bool two_launches = mfma_supported(a) && sgmv_supported(a) && sgmv_workspace_ok(a);
    const bool one_launch = mfma_supported(a) && wide_supported(a) && wide_pays(a) && !knobs().no_wide;
    if (!vec) form = MLORA_FORM_TOKEN;
    else if (one_launch && !(small_tiles && small_batch(a, true))) form = MLORA_FORM_WIDE;
    else if (!one_launch && two_launches && !(small_tiles && small_batch(a, false))) form = MLORA_FORM_SGMV;
    else if (small_tiles) form = MLORA_FORM_SPLIT;
    else form = MLORA_FORM_BGMV;
  }
  // the split form where it pays (a large A[slot]) and shape and workspace allow it, else one
  // workgroup per (tile, column range)
  if (form == MLORA_FORM_SPLIT && a->form != MLORA_FORM_SPLIT &&
      (knobs().no_split || !split_supported(a) || ((static_cast<long long>(a->r) * a->k < knobs().split_min_rk || a->num_tokens > knobs().split_max_tokens) && knobs().force_form != MLORA_FORM_SPLIT)))
    form = MLORA_FORM_MFMA;
  // small tiles with the grid laid over the slots where the shape allows it and slot ids are few.
  // Also where the split form would be taken: at K = 4096 the slot-major kernel shares K out between
  // the workgroups of a tile itself (down, decode batch, us per call, slot-major / split form:
  // rank 32: 8.1 / 10.6, rank 64: 10.7 / 17.0).
  if ((form == MLORA_FORM_MFMA || form == MLORA_FORM_SPLIT) && a->form == MLORA_FORM_AUTO && knobs().force_form != MLORA_FORM_MFMA &&
      knobs().force_form != MLORA_FORM_SPLIT && slot_supported(a) && slot_major_pays(a))
    form = MLORA_FORM_SLOT;
  // long-segment batches in one launch, on request
  if (form == MLORA_FORM_SGMV && a->form == MLORA_FORM_AUTO && knobs().force_form != MLORA_FORM_SGMV && knobs().auto_fused && fused_supported(a))
    form = MLORA_FORM_FUSED;
  switch (form) {
    case MLORA_FORM_TOKEN:
      return launch_token_add(a);
    case MLORA_FORM_BGMV:
      if ((a->effective_rank || !exact_rank(a->r)) && a->form == MLORA_FORM_AUTO) return launch_token_add(a);  // the vector-ALU tiles read whole rank-r rows
      if (!exact_rank(a->r)) { set_error("mlora_add_lora: the BGMV form takes ranks 8, 16, 32 and 64"); return MLORA_E_UNSUPPORTED; }
      if (a->effective_rank) { set_error("mlora_add_lora: the BGMV form does not take effective_rank"); return MLORA_E_UNSUPPORTED; }
      if (!vec) { set_error("mlora_add_lora: BGMV form needs 16-bit elements, a plan, rank in {8,16,32,64} and 16-byte aligned rows"); return MLORA_E_UNSUPPORTED; }
      return launch_bgmv(a, /*include_long=*/true);
    case MLORA_FORM_WIDE:
      if (!vec || !mfma_supported(a) || !wide_supported(a)) {
        set_error("mlora_add_lora: the one-launch form over 64-token tiles needs 16-bit elements, a plan, a rank of 8, 16, 32 or 64, K %% 128 == 0 "
                  "and no empty slice");
        return MLORA_E_UNSUPPORTED;
      }
      return launch_wide(a);
    case MLORA_FORM_SGMV:
    case MLORA_FORM_FUSED:
    case MLORA_FORM_SPLIT:
    case MLORA_FORM_SLOT:
    case MLORA_FORM_MFMA: {
      if (!vec || !mfma_supported(a)) { set_error("mlora_add_lora: MFMA forms need 16-bit elements, a plan, a rank that is a multiple of 8 up to 64 and K %% 32 == 0"); return MLORA_E_UNSUPPORTED; }
      if (form == MLORA_FORM_MFMA) return launch_decode(a, /*include_long=*/true);
      if (form == MLORA_FORM_SLOT) {
        if (!slot_supported(a)) {
          set_error("mlora_add_lora: the slot-major form needs one or two non-empty slices and K = 1024 (three at an exact rank with column "
                    "ranges of at most 512 columns), or K = 4096 with rank <= 16 or with one slice of at most 4096 columns and an "
                    "initialised workspace");
          return MLORA_E_UNSUPPORTED;
        }
        return launch_slot(a, trusted_workspace);
      }
      if (form == MLORA_FORM_SPLIT) {
        if (!split_supported(a)) {
          set_error("mlora_add_lora: the split form needs a rank of 8, 16, 32 or 64, K %% 512 == 0, at most 8 K parts, no empty slice and a 256-byte aligned "
                    "workspace of at least %d bytes whose exchange area holds every tile's partial sums", MLORA_WORKSPACE_HEAD_BYTES);
          return MLORA_E_UNSUPPORTED;
        }
        return launch_split(a, /*include_long=*/true, trusted_workspace);
      }
      if (!sgmv_supported(a)) { set_error("mlora_add_lora: SGMV form needs K %% 128 == 0 and a rank of 8, 16, 32 or 64"); return MLORA_E_UNSUPPORTED; }
      if (!sgmv_workspace_ok(a)) {
        set_error("mlora_add_lora: SGMV form needs a 16-byte aligned workspace of %zu bytes and no empty slice",
                  sgmv_workspace_bytes(a->num_tokens, a->num_slices, a->r, a->dtype));
        return MLORA_E_INVALID;
      }
      if (form == MLORA_FORM_FUSED) {
        if (!fused_supported(a)) {
          set_error("mlora_add_lora: the one-launch long-segment form needs K %% 256 == 0, at most %d groups of tiles and a workspace "
                    "whose head holds their seals", kWsTiles);
          return MLORA_E_UNSUPPORTED;
        }
        return launch_fused(a, trusted_workspace);
      }
      return launch_sgmv(a);
    }
  }
  set_error("mlora_add_lora: unreachable form %d", form);
  return MLORA_E_INVALID;
}

}  // namespace

// ---- the entry point that allocates nothing --------------------------------------------------
// Scratch of mlora_add_lora_static: part of the library's device image, so every GPU the
// library runs on holds its own copy at its own address from module load until the process ends.
// In host code the name `scratch` is only a handle for hipGetSymbolAddress; the address kernels
// and copies may use is the one that call returns, looked up once per device.
static __device__ __align__(256) unsigned char scratch[MLORA_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU (nullptr: not looked up yet)
std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch`; nullptr (and the error text set) on failure.
void* static_scratch(hipStream_t stream) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("mlora_add_lora_static: cannot identify the current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    // The look-up may load the code object, which a stream capture in progress does not survive:
    // the first call on a device has to be made outside any capture (one with num_tokens = 0 will do).
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) == hipSuccess && status == hipStreamCaptureStatusActive) {
      set_error("mlora_add_lora_static: the first call on a device must be made outside stream capture (call once with num_tokens = 0 before capturing)");
      return nullptr;
    }
    (void)hipGetLastError();
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      set_error("mlora_add_lora_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int mlora_add_lora_static(const MloraAddArgs* a) {
  if (!a) { set_error("mlora_add_lora_static: NULL args"); return MLORA_E_INVALID; }
  if (a->num_tokens < 0 || a->num_slices < 0 || a->r < 0) { set_error("mlora_add_lora_static: negative size"); return MLORA_E_INVALID; }
  const unsigned long long one_copy = 4ull * static_cast<unsigned long long>(a->num_tokens) * static_cast<unsigned long long>(a->num_slices) *
                                      static_cast<unsigned long long>(a->r);
  if (one_copy > MLORA_STATIC_SCRATCH_BYTES - MLORA_WORKSPACE_HEAD_BYTES) {
    set_error("mlora_add_lora_static: num_tokens x num_slices x r x 4 = %llu bytes exceed the static scratch of %u bytes behind its head (use mlora_add_lora with a workspace)",
              one_copy, static_cast<unsigned>(MLORA_STATIC_SCRATCH_BYTES - MLORA_WORKSPACE_HEAD_BYTES));
    return MLORA_E_TOO_LARGE;
  }
  void* ptr = static_scratch(static_cast<hipStream_t>(a->stream));
  if (!ptr) return MLORA_E_INVALID;
  MloraAddArgs b = *a;
  b.workspace = ptr;
  b.workspace_bytes = MLORA_STATIC_SCRATCH_BYTES;
  // The array starts out zeroed (it is part of the loaded image) and only this library's kernels
  // ever write it, so its head is always either in the initial state or as a launch left it.
  return add_lora_impl(&b, /*trusted_workspace=*/true);
}

extern "C" size_t mlora_add_workspace_bytes(int32_t num_tokens, int32_t num_slices, int32_t r, int32_t dtype) {
  if (num_tokens <= 0 || num_slices <= 0 || r <= 0) return 0;
  return sgmv_workspace_bytes(num_tokens, num_slices, r, dtype);  // head + room for every K part of the intermediate
}

extern "C" int mlora_workspace_init(void* workspace, int64_t workspace_bytes, void* stream) {
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255)) { set_error("mlora_workspace_init: workspace must be 256-byte aligned"); return MLORA_E_INVALID; }
  if (workspace_bytes < MLORA_WORKSPACE_HEAD_BYTES) {
    set_error("mlora_workspace_init: %lld bytes are fewer than MLORA_WORKSPACE_HEAD_BYTES = %d", static_cast<long long>(workspace_bytes), MLORA_WORKSPACE_HEAD_BYTES);
    return MLORA_E_INVALID;
  }
  return workspace_init(workspace, static_cast<hipStream_t>(stream));
}

extern "C" uint64_t mlora_stream_capture_id(void* stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long id = 0;
  if (hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &status, &id) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return status == hipStreamCaptureStatusActive ? static_cast<uint64_t>(id) : 0;
}

extern "C" void mlora_reload_knobs(void) { ++g_knob_generation; }

extern "C" int mlora_abi_version(void) { return MLORA_ABI_VERSION; }

extern "C" const char* mlora_last_error(void) { return g_error; }

extern "C" const char* mlora_build_info(void) {
  return "mlora gfx950 (wave64; small tiles: MFMA 16x16x32 or dot2 + wave reductions; big tiles: MFMA 16x16x32 shrink + expand) built " __DATE__ " " __TIME__;
}
