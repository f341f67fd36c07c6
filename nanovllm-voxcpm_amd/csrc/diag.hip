// Entry points of the diagnostic variants of the library (include/mlora_diag.h): none of them has a
// counterpart in the reference and none is part of the product library.
#include "common.h"
#include "launch.h"
#include "mlora_diag.h"

using namespace mlora;

extern "C" int mlora_trace_set(void* buf) {
#ifdef MLORA_TRACE
  decode_trace_set(buf);
  slot_trace_set(buf);
  split_trace_set(buf);
  fused_trace_set(buf);
  sgmv_trace_set(buf);
  wide_trace_set(buf);
  return 0;
#else
  (void)buf;
  set_error("mlora_trace_set: this library was built without MLORA_TRACE (make trace builds the variant that records timelines)");
  return MLORA_E_UNSUPPORTED;
#endif
}
