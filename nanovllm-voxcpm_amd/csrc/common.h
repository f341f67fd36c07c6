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

// ---- matrix-core products (fp32 accumulate) -------------------------------------------------
// 16x16x32: operand lane l holds row (or column) l % 16, elements 8 * (l / 16) .. + 7 of the
// contraction; the result lane holds rows 4 * (l / 16) .. + 3 of column l % 16.
template <typename T> struct Mma;
template <> struct Mma<__bf16> {
  static __device__ __forceinline__ f32x4 run(const Pack8& a, const Pack8& b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.bf, b.bf, c, 0, 0, 0);
  }
};
template <> struct Mma<_Float16> {
  static __device__ __forceinline__ f32x4 run(const Pack8& a, const Pack8& b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.hf, b.hf, c, 0, 0, 0);
  }
};

// 16x16x16 variant (four operand elements per lane): for rank 16 the contraction of the
// expand is exactly sixteen long, so no lane fetches B elements it would multiply by zero.
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));
template <typename T> struct Mma16;
template <> struct Mma16<__bf16> {
  static __device__ __forceinline__ f32x4 run(uint2 a, uint2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
};
template <> struct Mma16<_Float16> {
  static __device__ __forceinline__ f32x4 run(uint2 a, uint2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h16x4, a), __builtin_bit_cast(h16x4, b), c, 0, 0, 0);
  }
};

// After a run of MFMAs that a branch can cut short (rank blocks or k-steps left out at run time),
// and before anything else reads the accumulators.  An MFMA's result may not be read by another
// kind of instruction for some cycles after its issue; the compiler keeps that distance along
// straight-line code, but where such a run is left through a branch that lands on the reading
// code it was seen to provide for the longest way there only: the last MFMA's result was read
// two instructions after it and came out incomplete or not, depending on where the code lay in
// memory (rank-64 buffers with an adapter of rank 16 or less: the last k-step of a K part went
// missing).  24 idle cycles cover the longest MFMA; the accumulators are operands so that none
// of their reads is moved ahead of them.
template <int N> __device__ __forceinline__ void mfma_settle(f32x4 (&acc)[N]) {
  static_assert(N >= 1 && N <= 4, "accumulator blocks");
  if constexpr (N == 1) asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+v"(acc[0]));
  else if constexpr (N == 2) asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+v"(acc[0]), "+v"(acc[1]));
  else if constexpr (N == 3) asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]));
  else asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]));
}

// Zero the elements of an eight-element chunk that hold ranks at or above `eff`; `first` is the
// rank of the chunk's element 0.
__device__ __forceinline__ void mask_ranks(Pack8& p, int first, int eff) {
  const int keep = eff - first;  // elements 0 .. keep - 1 stay
#pragma unroll
  for (int d = 0; d < 4; ++d) p.u[d] &= (2 * d < keep ? 0x0000ffffu : 0u) | (2 * d + 1 < keep ? 0xffff0000u : 0u);
}

// Rank of the adapter in a slot without a dependent fetch.  The slot of a tile is only known once
// its record has arrived, and a fetch that waits for it costs a whole trip to memory in a kernel
// that lives for a handful of trips.  The per-slot rank vector is small, so every lane requests
// entries lane, lane + 64, ... of it together with the record (their addresses depend on nothing),
// and the slot's entry is picked out of the registers afterwards.  Vectors beyond 256 slots fall
// back to the dependent fetch.
struct RankPrefetch {
  int v[4];
};
__device__ __forceinline__ RankPrefetch rank_prefetch(const int32_t* __restrict__ eff_rank, int num_slots, int lane) {
  RankPrefetch p;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + 64 * j;
    p.v[j] = (eff_rank && 64 * j < num_slots) ? eff_rank[i < num_slots ? i : num_slots - 1] : 0;
  }
  return p;
}
__device__ __forceinline__ int rank_pick(const RankPrefetch& p, const int32_t* __restrict__ eff_rank, int num_slots, int slot, int R) {
  if (!eff_rank) return R;
  int e;
  if (num_slots <= 256) {
    const int s = __builtin_amdgcn_readfirstlane(slot);  // the same in every lane
    const int j = s >> 6;
    const int word = j == 0 ? p.v[0] : j == 1 ? p.v[1] : j == 2 ? p.v[2] : p.v[3];
    e = __builtin_amdgcn_readlane(word, s & 63);
  } else {
    e = eff_rank[slot];
  }
  return e < 0 ? 0 : e > R ? R : e;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// ---- plan workspace layout ------------------------------------------------------------
// int32 words:  header | sorted_idx[T] | counts[L+1] | offsets[L+2] | small tiles | big tiles | big-tile rows |
//               records by slot | records of the further small tiles
// Small tiles are 32-word records (128-byte aligned), big tiles four words, their row lists 64 words; see mlora.h.
struct PlanLayout {
  int sorted_off, counts_off, offsets_off, small_off, big_off, bigrows_off, cap_small, cap_big;
  int slotrec_off, cap_slotrec, over_off, cap_over, total_words;
};

__host__ __device__ inline int round_up4(int v) { return (v + 3) & ~3; }

// Where the 64-token tiles lie in their list.  The list is cut into eight equal blocks, one per
// XCD: workgroup (x, ., z) of a launch takes place x * (capacity / 8) + z.  The tiles are sorted by
// slot; runs of consecutive tiles go to the blocks in turn (run i to block i % 8, behind the runs
// the block already holds).  With long runs the tiles of a slot meet few XCDs and its weights are
// fetched into few L2s; with runs of one tile the XCDs take the tiles in turn.  Workgroups are
// dispatched layer by layer (z), every XCD's z-th tile together, so a layer costs what its most
// expensive tile costs: runs may be as long as the slots' segments are (then a layer holds tiles
// of the same kind, mostly full ones), and no longer than an eighth of the list.
//   run length: the tiles split into 8 k runs, k the smallest for which a run is no longer than
//   the average number of tiles of a slot that has any.
__host__ __device__ inline int big_tile_run(int n_big, int slots_with_tiles) {
  if (n_big <= 0) return 1;
  const int avg = n_big / (slots_with_tiles > 0 ? slots_with_tiles : 1);  // >= 1
  const int k = (n_big + 8 * avg - 1) / (8 * avg);
  return (n_big + 8 * k - 1) / (8 * k);
}
__host__ __device__ inline int big_tile_place(int t, int run, int cap_big) {
  const int i = t / run;
  return (i & 7) * (cap_big >> 3) + (i >> 3) * run + t % run;
}
// Places for at most `most` tiles: a block holds ceil(runs / 8) runs, less than most / 8 + run
// places, and a run is at most ceil(most / (8 k)) with k runs a block: most / 8 + sqrt(most / 8) + 1
// places bound both; a multiple of 32.
__host__ __device__ inline int big_tile_capacity(int most) {
  int root = 1;
  while (root * root * 8 < most) ++root;
  return (most + 8 * (root + 2) + 31) & ~31;
}

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
  // groups of up to four tiles, eight blocks abreast (one per XCD), each block with room for an
  // eighth of the tiles and a run of them (big_tile_place)
  p.cap_big = big_tile_capacity(T / MLORA_TILE_BIG + segs);
  p.bigrows_off = p.big_off + MLORA_BIG_TILE_WORDS * p.cap_big;  // (a multiple of 32 words again)
  // the small tiles once more, by slot: one record per slot id, then one per further tile (a
  // further tile has sixteen tokens of its slot in front of it, so T / 16 bounds their number)
  p.slotrec_off = p.bigrows_off + MLORA_TILE_BIG * p.cap_big;
  p.cap_slotrec = (L + 7) & ~7;
  p.over_off = p.slotrec_off + MLORA_SMALL_TILE_WORDS * p.cap_slotrec;
  p.cap_over = (T / MLORA_TILE_SMALL + 7) & ~7;
  p.total_words = p.over_off + MLORA_SMALL_TILE_WORDS * p.cap_over;
  return p;
}

// A launch that finds its plan built for another batch shape (or not built at all) leaves y as it
// was; its first workgroup counts the launch in the plan's header (MLORA_PLAN_REJECTED), the one
// word of a plan that the apply kernels write.  Called on the way out only: nothing of it stands
// in front of a working workgroup's loads.
__device__ __forceinline__ void count_rejected_plan(const int32_t* plan, bool header_ok) {
  if (!header_ok && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
    atomicAdd(const_cast<int32_t*>(plan) + MLORA_PLAN_REJECTED, 1);
}

// ---- workspace head (see MLORA_WORKSPACE_HEAD_BYTES in mlora.h) -------------------------------
// uint32 words:  [0] signature | [1] waits that ran out (diagnostic) | ... ; at byte kWsTileOff the
// {generation, arrivals} pair of the workspace (every workgroup of a split or one-launch
// long-segment grid reports once when it is done, the last one advances the generation; the rest of
// the 8 KiB behind it is reserved); at byte kWsXchgOff the exchange area of the split form: 64-bit
// words {fp32 bits, tag}, valid when tag == generation + 1.  One generation for the whole
// workspace: whatever an earlier launch left anywhere in the area, in whatever layout, carries a
// tag below the current one.
constexpr uint32_t kWsMagic = 0x4d4c5733u;  // "MLW3"
// Third word of the {generation, arrivals} pair: generation ^ kWsGenCheck, rewritten with every
// advance of the generation.  A head is believed only if signature, this word and an arrival count
// below the grid size all fit: memory that once was a workspace and was handed out again in between
// can keep the signature while the pair holds something else, and a generation that never advances
// would make the next launch accept what the last one left.
constexpr uint32_t kWsGenCheck = 0x9e3779b9u;
__device__ __forceinline__ bool ws_state_ok(uint32_t signature, uint32_t generation, uint32_t arrivals, uint32_t check, uint32_t grid) {
  return signature == kWsMagic && check == (generation ^ kWsGenCheck) && arrivals < grid;
}
constexpr int kWsTimeoutsWord = 1;
constexpr int kWsTileOff = 256;
constexpr int kWsTiles = 1024;
constexpr int kWsXchgOff = 16384;
constexpr int kWsXchgBytes = 4 << 20;
// behind the exchange area: one 64-bit seal per (unit, shrink role) of the one-launch
// long-segment form: {generation of the unit + 1, XCD of the writer}
constexpr int kWsSealBytes = 64 << 10;
constexpr int kWsSealOff = kWsXchgOff + kWsXchgBytes;
static_assert(kWsTileOff + 8 * kWsTiles <= kWsXchgOff, "tile state overlaps the exchange area");
static_assert(kWsSealOff + kWsSealBytes == MLORA_WORKSPACE_HEAD_BYTES, "head size");

// The XCD (accelerator die) this wavefront runs on: bits 3:0 of hardware register XCC_ID (id 20).
__device__ __forceinline__ uint32_t xcc_id() { return __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15u; }

// ---- in-kernel timeline (builds with -DMLORA_TRACE only) ---------------------------------------
// MLORA_STAMP(i) makes thread 0 of a workgroup record the 100 MHz clock in slot i of the
// workgroup's row of the buffer handed to mlora_trace_set (16 slots per workgroup, workgroups in
// dispatch order).  Without MLORA_TRACE it expands to nothing.
#ifdef MLORA_TRACE
#define MLORA_TRACE_DECL static __device__ unsigned long long* trace_buf = nullptr;
#define MLORA_STAMP(i)                                                                                       \
  do {                                                                                                       \
    if (threadIdx.x == 0 && trace_buf)                                                                       \
      trace_buf[(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * 16ull + (i)] = wall_clock64(); \
  } while (0)
// the same by thread `t` of the workgroup
#define MLORA_STAMP_AT(i, t)                                                                                 \
  do {                                                                                                       \
    if (threadIdx.x == (t) && trace_buf)                                                                     \
      trace_buf[(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * 16ull + (i)] = wall_clock64(); \
  } while (0)
#else
#define MLORA_TRACE_DECL
#define MLORA_STAMP(i) \
  do {                 \
  } while (0)
#define MLORA_STAMP_AT(i, t) \
  do {                       \
  } while (0)
#endif

// ---- error reporting --------------------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

}  // namespace mlora
