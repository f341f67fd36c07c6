/*
 * mlora_diag.h - measurement and test aids of the MI355X multi-LoRA library.  Nothing here has a
 * counterpart in the reference and nothing here is needed to use the library: include/mlora.h is
 * the product's C-ABI.
 *
 * mlora_probe_launch and mlora_trace_set are exported by the diagnostic variants only
 * (libmlora_gfx950_diag.so from `make diag`, libmlora_gfx950_trace.so from `make trace`).
 * mlora_reload_knobs is exported by every variant: the test-suite changes MLORA_* variables
 * between tests of one process.
 */
#ifndef MLORA_DIAG_H_
#define MLORA_DIAG_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Diagnostic knobs (the MLORA_* environment variables) are read once per process and kept;
 * this makes the next call read them again. */
void mlora_reload_knobs(void);

/* Launches of known cost: kind 0 enqueues a kernel that does nothing with the given grid and
 * workgroup size (what a launch costs by itself); kind 1 a read-modify-write stream over `bytes`
 * of 16-bit elements at `buf` (every element read, incremented, written back once: the access
 * pattern of y); kind 2 a read-only stream over them; kind 3 a kernel of the given grid whose
 * workgroups each write the number of the XCD they run on to `buf` (int32 per workgroup, linear
 * workgroup order: the placement the kernels' grids of x extent 8 rely on can be checked). */
int mlora_probe_launch(void* stream, int32_t kind, void* buf, int64_t bytes, int32_t grid_x, int32_t grid_y, int32_t grid_z,
                       int32_t threads);

/* In-kernel timelines.  The variant built with `make trace` records, per workgroup of the apply
 * kernels, up to 16 readings of the 100 MHz clock at fixed points of the kernel into `buf`
 * (uint64 [workgroups][16], device memory the caller zeroes; NULL switches recording off).  The
 * diag variant returns MLORA_E_UNSUPPORTED. */
int mlora_trace_set(void* buf);

#ifdef __cplusplus
}
#endif
#endif /* MLORA_DIAG_H_ */
