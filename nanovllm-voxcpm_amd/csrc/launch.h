// Internal launch entry points shared by the C-ABI front door.
#pragma once

#include <hip/hip_runtime.h>

#include "mlora.h"

namespace mlora {

int env_int(const char* name, int fallback);

// Ranks the kernels are instantiated for.  Buffers of another rank that is a multiple of eight and
// at most 64 (24, 40, 48, 56) run on the next instance up in the small-tile kernels, with the
// buffers' rank as the run-time stride and everything beyond it masked as for an adapter of lower
// rank; the other forms take exact ranks only.
inline bool exact_rank(int r) { return r == 8 || r == 16 || r == 32 || r == 64; }
inline bool padded_rank(int r) { return r >= 8 && r <= 64 && r % 8 == 0; }
inline int compute_rank(int r) { return r <= 8 ? 8 : r <= 16 ? 16 : r <= 32 ? 32 : 64; }
// Diagnostic knobs are read from the environment once and kept; mlora_reload_knobs() advances
// this number, and a holder whose copy is older reads its variables again.
int knob_generation();

// token.hip: one workgroup per token; needs only token_to_slot.
int launch_token_add(const MloraAddArgs* a);

// bgmv.hip: small tiles (<= 16 tokens of one slot) on the vector ALU.  include_long selects
// whether the small tiles of segments at or above the threshold are walked too.
int launch_bgmv(const MloraAddArgs* a, bool include_long);

// decode.hip: the same small tiles with both products on the matrix cores, one workgroup per
// (tile, column range).
bool decode_supported(const MloraAddArgs* a);  // x and y below 2 GiB each
int launch_decode(const MloraAddArgs* a, bool include_long);

// slot.hip: the same small tiles, the grid laid over the slots: weights are requested from the
// workgroup index alone, before the slot's record has arrived.
bool slot_supported(const MloraAddArgs* a);
int slot_k_parts(const MloraAddArgs* a);  // 4 when the workgroups of a tile would share K out, else 1
int launch_slot(const MloraAddArgs* a, bool trusted_workspace);

// split.hip: the same small tiles, producers and consumers of the intermediate in one launch.
// trusted_workspace: the head of the workspace is known to be in its initial or a left-behind
// state without carrying the signature (the library's own zero-initialised array).
bool split_supported(const MloraAddArgs* a);
int launch_split(const MloraAddArgs* a, bool include_long, bool trusted_workspace);
int workspace_init(void* workspace, hipStream_t stream);

// sgmv.hip: 64-token MFMA tiles of the segments at or above the threshold, as a shrink launch
// and an expand launch that meet in the caller's workspace.
bool sgmv_supported(const MloraAddArgs* a);
bool sgmv_workspace_ok(const MloraAddArgs* a);
size_t sgmv_workspace_bytes(int num_tokens, int num_slices, int r, int dtype);
int launch_sgmv(const MloraAddArgs* a);

// fused.hip: the same tiles, shrink and expand in one launch (workgroups of a unit exchange the
// intermediate through the workspace under seals kept in its head).
bool fused_supported(const MloraAddArgs* a);
int launch_fused(const MloraAddArgs* a, bool trusted_workspace);

// wide.hip: the same tiles, one launch, one workgroup per (tile, column range) doing both products.
bool wide_supported(const MloraAddArgs* a);
bool wide_pays(const MloraAddArgs* a);
int launch_wide(const MloraAddArgs* a);

// in-kernel timeline of trace builds (no-ops otherwise)
void decode_trace_set(void* buf);
void slot_trace_set(void* buf);
void split_trace_set(void* buf);
void fused_trace_set(void* buf);
void sgmv_trace_set(void* buf);
void wide_trace_set(void* buf);

}  // namespace mlora
