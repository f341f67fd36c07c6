// Internal launch entry points shared by the C-ABI front door.
#pragma once

#include "mlora.h"

namespace mlora {

int env_int(const char* name, int fallback);

// token.hip: one workgroup per token; needs only token_to_slot.
int launch_token_add(const MloraAddArgs* a);

// bgmv.hip: small tiles (<= 16 tokens of one slot) on the vector ALU.  include_long selects
// whether the small tiles of segments at or above the threshold are walked too.
int launch_bgmv(const MloraAddArgs* a, bool include_long);

// decode.hip: the same small tiles with both products on the matrix cores.
int launch_decode(const MloraAddArgs* a, bool include_long);
size_t decode_workspace_bytes(int r);

// sgmv.hip: 64-token MFMA tiles of the segments at or above the threshold, as a shrink launch
// and an expand launch that meet in the caller's workspace.
bool sgmv_supported(const MloraAddArgs* a);
bool sgmv_workspace_ok(const MloraAddArgs* a);
size_t sgmv_workspace_bytes(int num_tokens, int num_slices, int r, int dtype);
int launch_sgmv(const MloraAddArgs* a);

}  // namespace mlora
