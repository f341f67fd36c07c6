// Shared device/host helpers for the gfx950 multi-LoRA apply kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mlora.h"

namespace mlora {

constexpr int kWave = 64;

// ---- element types --------------------------------------------------------------------
template <int DT> struct Elem;
template <> struct Elem<MLORA_DTYPE_F32> { using type = float; };
template <> struct Elem<MLORA_DTYPE_F16> { using type = _Float16; };
template <> struct Elem<MLORA_DTYPE_BF16> { using type = __bf16; };

template <typename T> __device__ __forceinline__ float to_f32(T v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return static_cast<T>(v); }

typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2;

// Eight 16-bit elements moved as one 128-bit word.
union Pack8 {
  i32x4 raw;
  bf16x8 bf;
  f16x8 hf;
  bf16x2 bf2[4];
  f16x2 hf2[4];
  uint32_t u[4];
};

__device__ __forceinline__ i32x4 load128(const void* p) { return *reinterpret_cast<const i32x4*>(p); }
__device__ __forceinline__ void store128(void* p, i32x4 v) { *reinterpret_cast<i32x4*>(p) = v; }

// Dot product of eight 16-bit pairs accumulated in fp32 with the packed dot2 instructions.
template <typename T> __device__ __forceinline__ float dot8(const Pack8& a, const Pack8& b, float acc);
template <> __device__ __forceinline__ float dot8<__bf16>(const Pack8& a, const Pack8& b, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(a.bf2[i], b.bf2[i], acc, false);
  return acc;
}
template <> __device__ __forceinline__ float dot8<_Float16>(const Pack8& a, const Pack8& b, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(a.hf2[i], b.hf2[i], acc, false);
  return acc;
}

// Unpack eight 16-bit elements to fp32.
template <typename T> __device__ __forceinline__ void unpack8(const Pack8& p, float (&out)[8]);
template <> __device__ __forceinline__ void unpack8<__bf16>(const Pack8& p, float (&out)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = __uint_as_float(p.u[i] << 16);
    out[2 * i + 1] = __uint_as_float(p.u[i] & 0xffff0000u);
  }
}
template <> __device__ __forceinline__ void unpack8<_Float16>(const Pack8& p, float (&out)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = static_cast<float>(p.hf[i]);
}
template <typename T> __device__ __forceinline__ void pack8(const float (&in)[8], Pack8& p);
template <> __device__ __forceinline__ void pack8<__bf16>(const float (&in)[8], Pack8& p) {
#pragma unroll
  for (int i = 0; i < 8; ++i) p.bf[i] = static_cast<__bf16>(in[i]);
}
template <> __device__ __forceinline__ void pack8<_Float16>(const float (&in)[8], Pack8& p) {
#pragma unroll
  for (int i = 0; i < 8; ++i) p.hf[i] = static_cast<_Float16>(in[i]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// ---- plan workspace layout ------------------------------------------------------------
// int32 words:  header | sorted_idx[T] | counts[L+1] | offsets[L+2] | small tiles | big tiles
// Small tiles are 32-word records (128-byte aligned), big tiles four words; see mlora.h.
struct PlanLayout {
  int sorted_off, counts_off, offsets_off, small_off, big_off, coop_off, cap_small, cap_big, total_words;
};

__host__ __device__ inline int round_up4(int v) { return (v + 3) & ~3; }

__host__ __device__ inline PlanLayout plan_layout(int T, int L) {
  PlanLayout p;
  const int segs = L < T ? L : T;
  p.sorted_off = MLORA_PLAN_HEADER_WORDS;
  p.counts_off = p.sorted_off + round_up4(T);
  p.offsets_off = p.counts_off + round_up4(L + 1);
  p.small_off = (p.offsets_off + round_up4(L + 2) + 31) & ~31;
  // capacities are multiples of eight: launches walk the tile lists in groups of eight (one
  // tile per XCD), and every record such a grid may touch has to exist
  p.cap_small = ((T + MLORA_TILE_SMALL - 1) / MLORA_TILE_SMALL + segs + 7) & ~7;
  p.big_off = p.small_off + MLORA_SMALL_TILE_WORDS * p.cap_small;
  p.cap_big = (T / MLORA_TILE_BIG + segs + 31) & ~31;  // groups of up to four tiles, eight groups abreast
  // arrival counters of the workgroups that share one small tile's shrink (zero between launches)
  p.coop_off = p.big_off + MLORA_BIG_TILE_WORDS * p.cap_big;
  p.total_words = p.coop_off + MLORA_COOP_SPLITS * p.cap_small;
  return p;
}

// ---- error reporting --------------------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

}  // namespace mlora
