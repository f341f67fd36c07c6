// Internal launch entry points shared by the C-ABI front door.
#pragma once

#include "mlora.h"

namespace mlora {

int env_int(const char* name, int fallback);

// token.hip: one workgroup per token; needs only token_to_slot.
int launch_token_add(const MloraAddArgs* a);

// bgmv.hip: small tiles (<= 8 tokens of one slot) from the plan.  include_long selects
// whether the small tiles of segments at or above the threshold are walked too.
int launch_bgmv(const MloraAddArgs* a, bool include_long);

// sgmv.hip: MFMA tiles.  all_segments additionally sends the short segments through the
// 16-row MFMA variant instead of leaving them to launch_bgmv.
bool sgmv_supported(const MloraAddArgs* a);
int launch_sgmv(const MloraAddArgs* a, bool all_segments);

}  // namespace mlora
