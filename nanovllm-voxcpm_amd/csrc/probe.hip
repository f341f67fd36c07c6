// Measurement aids with no counterpart in the reference: launches whose cost is known by
// construction, so that a benchmark can state what one dependent launch costs on the machine it
// runs on and what rate a plain stream over HBM reaches there, beside the numbers of the real
// kernels.
#include "common.h"
#include "launch.h"
#include "mlora_diag.h"

namespace mlora {

namespace {

// kind 0: a kernel that does nothing (any grid): cost of a launch by itself.
__global__ void probe_empty_kernel() {}

// kind 1: read-modify-write stream, 128-bit accesses: every 16-bit element of the buffer is read,
// incremented in fp32 and written back once (the access pattern of y in the apply kernels).
__global__ __launch_bounds__(256) void probe_rmw_kernel(i32x4* __restrict__ buf, int64_t chunks) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < chunks; i += stride) {
    Pack8 p;
    p.raw = buf[i];
    float f[8];
    unpack8<__bf16>(p, f);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] += 1.0f;
    pack8<__bf16>(f, p);
    buf[i] = p.raw;
  }
}

// kind 2: read-only stream (sum kept from being optimised away by a never-true store).
__global__ __launch_bounds__(256) void probe_read_kernel(const i32x4* __restrict__ buf, int64_t chunks, int* sink) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  int acc = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < chunks; i += stride) {
    const i32x4 v = buf[i];
    acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (acc == 0x5a5a5a5a && sink) *sink = acc;
}

// kind 3: every workgroup of a (grid_x, grid_y, grid_z) grid records the XCD it runs on (one int32
// per workgroup, in linear workgroup order): what the kernels assume about grids whose x extent
// is 8 (blockIdx.x names the XCD) can be checked on the machine at hand.
__global__ void probe_xcd_kernel(int32_t* __restrict__ out) {
  if (threadIdx.x == 0) out[blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)] = static_cast<int32_t>(xcc_id());
}

}  // namespace

}  // namespace mlora

using namespace mlora;

extern "C" int mlora_probe_launch(void* stream, int32_t kind, void* buf, int64_t bytes, int32_t grid_x, int32_t grid_y, int32_t grid_z,
                                  int32_t threads) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (kind == 0) {
    if (grid_x < 1 || grid_y < 1 || grid_z < 1 || threads < 1 || threads > 1024) { set_error("mlora_probe_launch: bad launch shape"); return MLORA_E_INVALID; }
    hipLaunchKernelGGL(probe_empty_kernel, dim3(grid_x, grid_y, grid_z), dim3(threads), 0, st);
    return check_launch("mlora_probe_launch(empty)");
  }
  if (kind == 3) {
    if (grid_x < 1 || grid_y < 1 || grid_z < 1 || threads < 1 || threads > 1024) { set_error("mlora_probe_launch: bad launch shape"); return MLORA_E_INVALID; }
    if (!buf || bytes < static_cast<int64_t>(grid_x) * grid_y * grid_z * 4) { set_error("mlora_probe_launch: one int32 per workgroup is needed"); return MLORA_E_INVALID; }
    hipLaunchKernelGGL(probe_xcd_kernel, dim3(grid_x, grid_y, grid_z), dim3(threads), 0, st, static_cast<int32_t*>(buf));
    return check_launch("mlora_probe_launch(xcd)");
  }
  if (kind != 1 && kind != 2) { set_error("mlora_probe_launch: unknown kind %d", kind); return MLORA_E_INVALID; }
  if (!buf || bytes < 16 || (reinterpret_cast<uintptr_t>(buf) & 15)) { set_error("mlora_probe_launch: a 16-byte aligned buffer is needed"); return MLORA_E_INVALID; }
  const int64_t chunks = bytes / 16;
  int64_t blocks = (chunks + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  if (kind == 1) hipLaunchKernelGGL(probe_rmw_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, static_cast<i32x4*>(buf), chunks);
  else hipLaunchKernelGGL(probe_read_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, static_cast<const i32x4*>(buf), chunks, static_cast<int*>(nullptr));
  return check_launch("mlora_probe_launch(stream)");
}
