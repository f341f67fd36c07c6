// Computes, for decode-sized batches, what the reference computes with a shrink launch, a
// temporary [slices, T, r] tensor and one or two expand launches
// (nanovllm_voxcpm/lora.py:291-381 driving lora_ops/triton_ops/lora_shrink_op.py:16-173,
// lora_expand_op.py:11-91 and kernel_utils.py:7-228): y_i[t] += (x[t] . A_i[s_t]^T) . B_i[s_t]^T * scaling.
//
// Split form: ONE launch in which the two products of a small tile (up to sixteen tokens of one
// slot) are done by different workgroups.
//   producer (tile, slice, K part)      fetches its part of the x rows and of A[slot], multiplies
//                                       (MFMA 16x16x32, eight or four wavefronts splitting the K
//                                       part), and publishes the 16 x r partial sums in the
//                                       workspace;
//   consumer (tile, slice, column range) requests the B[slot] rows and y rows of its columns at
//                                       once, picks the partial sums up as soon as they are
//                                       there, and expands.
// A decode launch moves a few MB; what bounds it is the latency chain of one workgroup and the
// rate at which one compute unit takes data in (about 20 bytes per cycle, cache hits included),
// not HBM.  When every column range repeats the shrink of its tile (the one-kernel form in
// decode.hip) each compute unit pulls x and A[slot] on top of its own B and y; here every operand
// element passes through exactly one compute unit and the launch spreads over several hundred
// small workgroups.
//
// The hand-over needs no counter on its critical path.  Every published 64-bit word carries the
// partial sum and a tag; the tag is the tile's generation + 1, read by producers and consumers
// alike at the start of the launch, so a consumer polls the data words themselves and accepts a
// word when its tag matches.  A workgroup that is done with the exchange area counts itself on
// the tile; the last one of a tile advances the tile's generation, which invalidates everything
// the launch left behind — nothing is ever cleared.  All workgroups of a tile run on one XCD
// (grid x = XCD), so tags, counts and data meet in that XCD's L2.
// Waiting is bounded: a consumer whose words are not there after `spin_ticks` of the 100 MHz
// clock computes the partial sums itself, with the producers' split of K and order of additions,
// so results never depend on timing and every workgroup exits whatever the others do.  The same
// path serves a workspace that was never initialised (no signature): nobody publishes, nobody
// waits.
#include "common.h"
#include "launch.h"

namespace mlora {

namespace {

constexpr int kNW = 8;          // wavefronts per workgroup
constexpr int kNT = kNW * kWave;
constexpr int kSpansAhead = 2;  // output spans per wavefront whose loads are issued up front
constexpr int kStageRow = 17;   // 16 chunks of 16 bytes + one of padding: operand reads hit every bank once

MLORA_TRACE_DECL

struct SplitSlices {
  const void* a[MLORA_MAX_SLICES];
  const void* b[MLORA_MAX_SLICES];
  int n[MLORA_MAX_SLICES];
  int y_col[MLORA_MAX_SLICES];
  int cons0[MLORA_MAX_SLICES + 1];  // consumer roles of slice s: [cons0[s], cons0[s + 1]), counted from the first consumer
};

typedef unsigned long long u64;

// Accesses to words that another workgroup of the same launch writes or reads.  Bits of `wide`
// select device scope (performed where all XCDs meet) for loads (1), stores (2) and counters (4);
// without them they are performed in the L2 of the XCD, which is where all workgroups of a tile run.
__device__ __forceinline__ u64 xload(const u64* p, int wide) {
  return (wide & 1) ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                    : __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void xstore(u64* p, u64 v, int wide) {
  if (wide & 2) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ uint32_t xadd(uint32_t* p, uint32_t v, int wide) {
  return (wide & 4) ? __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                    : __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void xstore32(uint32_t* p, uint32_t v, int wide) {
  if (wide & 4) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// NWP: wavefronts of a producer that take part in the shrink; a K part is NWP * 128 columns.
template <typename T, int R, int NWP, bool MASKED>
__global__ __launch_bounds__(kNT) void split_kernel(const int32_t* __restrict__ plan, const void* __restrict__ xv, void* __restrict__ yv_,
                                                    int64_t xs, int64_t ys, uint32_t* __restrict__ ws, int small_off, int T_, int K,
                                                    int num_slots, float scaling, int include_long, int S, int P, int W, int spin_ticks,
                                                    int wide, int trusted, int sym, const int32_t* __restrict__ eff_rank, SplitSlices sl) {
  constexpr int RB = (R + 15) / 16;      // 16-rank blocks of the shrink output
  constexpr int KSTEPS = (R + 31) / 32;  // MFMA k-steps of the expand
  constexpr int HSTRIDE = R + 8;         // padded LDS row of the intermediate
  constexpr int WORDS = 16 * R;          // partial sums of one (tile, slice, K part)
  constexpr int WPT = (WORDS + kNT - 1) / kNT;  // of which a thread sums up this many
  constexpr int WPL = R / 4;             // words per lane when one wavefront fetches a part
  constexpr bool K16 = R == 16;          // expand on the 16x16x16 MFMA: 64-bit operand pieces

  __shared__ __attribute__((aligned(16))) float s_red[NWP * RB * 256];
  __shared__ __attribute__((aligned(16))) T s_hi[16 * HSTRIDE];
  __shared__ __attribute__((aligned(16))) T s_lo[16 * HSTRIDE];
  __shared__ __attribute__((aligned(16))) i32x4 s_stage[kNW * 16 * kStageRow];
  __shared__ int s_ok;

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;
  const int tile = blockIdx.z * 8 + blockIdx.x;  // blockIdx.x is the XCD
  const int role = blockIdx.y;
  MLORA_STAMP(0);  // first instruction

  // ---- round trip 1: everything whose address depends on the workgroup index only ---------------
  const int32_t* rec = plan + small_off + tile * MLORA_SMALL_TILE_WORDS;  // tile < capacity: in bounds
  const i32x4 rows4 = *reinterpret_cast<const i32x4*>(rec + MLORA_SMALL_TILE_ROWS + 4 * lg);  // tokens 4*lg .. 4*lg+3
  const i32x4 rec0 = *reinterpret_cast<const i32x4*>(rec);       // slot, count, start, 0
  const i32x4 hdr0 = *reinterpret_cast<const i32x4*>(plan);      // magic, T, L, ...
  const i32x4 hdr1 = *reinterpret_cast<const i32x4*>(plan + 4);  // ..., short tiles
  const i32x4 hdr2 = *reinterpret_cast<const i32x4*>(plan + 8);  // long small tiles, ...
  const uint32_t signature = ws[0];
  const RankPrefetch ranks = rank_prefetch(MASKED ? eff_rank : nullptr, num_slots, lane);
  // {generation, arrivals} of the workspace: one pair for the whole launch, so that every tagged
  // word any earlier launch left anywhere in the exchange area (whatever its layout was) carries a
  // tag below this launch's
  uint32_t* const tstate = ws + kWsTileOff / 4;
  const uint32_t tag = tstate[0] + 1u;
  const uint32_t arrivals0 = tstate[1], gen_check = tstate[2];
  const int slot = rec0[0], m = rec0[1];
  const int n_tiles = hdr1[MLORA_PLAN_TILES_SHORT - 4] + hdr2[MLORA_PLAN_TILES_LONG_SMALL - 8] * include_long;
  // One exit test, the same for every workgroup of a tile
  const int usable = int(hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE) & int(hdr0[MLORA_PLAN_NUM_TOKENS] == T_) &
                     int(hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots) & int(tile < n_tiles) & int(m > 0) & int(slot >= 0) &
                     int(slot < num_slots);
  // the exchange area can be used: the head is in the state a launch (or the initialisation) left it in
  const bool xok = trusted | ws_state_ok(signature, tag - 1u, arrivals0, gen_check, gridDim.x * gridDim.y * gridDim.z);
  // Every workgroup of the grid reports exactly once that it is done with the exchange area (also
  // the ones without work); the last one advances the generation.  Counted by the last wavefront,
  // which has the least other work: the count comes back from the memory system long after it was
  // sent, and whoever sent it has to wait for it.
  auto count_done = [&]() {
    if (xok && tid == kNT - kWave) {
      const uint32_t before = xadd(tstate + 1, 1u, wide);
      if (before + 1u == gridDim.x * gridDim.y * gridDim.z) {
        const uint32_t next = tag == 0xffffffffu ? 0u : tag;  // so that generation + 1, the next tag, is never 0
        xstore32(tstate + 1, 0u, wide);
        xstore32(tstate + 2, next ^ kWsGenCheck, wide);
        xstore32(tstate, next, wide);
      }
    }
  };
  if (!usable) {
    count_rejected_plan(plan, hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE && hdr0[MLORA_PLAN_NUM_TOKENS] == T_ &&
                                  hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots);
    count_done();
    return;
  }
  MLORA_STAMP(1);  // tile record, plan header and generation are here

  // rank of the adapter in this slot (requested together with the record, see rank_prefetch)
  // (MASKED = false is the instance for callers that gave no rank vector: eff is the constant R
  // there and every test on it below folds away)
  const int eff = MASKED ? rank_pick(ranks, eff_rank, num_slots, slot, R) : R;
  if (MASKED && eff == 0) {  // nothing resident: the same for every workgroup of the tile
    count_done();
    return;
  }
  const int rb_n = MASKED ? (eff + 15) >> 4 : RB;  // 16-rank blocks of A in use

  // Roles.  Asymmetric launch: S * P producers (slice, K part), then the consumers (slice, column
  // range of W columns).  Symmetric launch (sym, chosen for long K): S * P workgroups, each
  // producer of its K part and consumer of the part-th column range of its slice, so that the
  // shrink's operands AND the expand's are spread over all of them.
  const bool producer = role < S * P;
  const bool consumer = sym || !producer;
  int slice, part = 0, n0 = 0, n1 = 0;
  if (producer) {
    slice = role / P;
    part = role - slice * P;
    if (sym) {
      const int ws_cols = ((sl.n[slice] + P - 1) / P + 63) & ~63;  // columns per part, whole 64-column spans
      n0 = part * ws_cols < sl.n[slice] ? part * ws_cols : sl.n[slice];
      n1 = n0 + ws_cols < sl.n[slice] ? n0 + ws_cols : sl.n[slice];
    } else if (!xok) {
      return;  // nobody would read what this workgroup publishes (and nobody counts)
    }
  } else {
    const int c = role - S * P;
    slice = 0;
#pragma unroll
    for (int i = 1; i < MLORA_MAX_SLICES; ++i) slice += int(i < S && c >= sl.cons0[i]);
    n0 = (c - sl.cons0[slice]) * W;
    n1 = n0 + W < sl.n[slice] ? n0 + W : sl.n[slice];
  }
  const int N = sl.n[slice];
  const T* const A = static_cast<const T*>(sl.a[slice]) + static_cast<int64_t>(slot) * R * K;
  u64* const xchg = reinterpret_cast<u64*>(reinterpret_cast<char*>(ws) + kWsXchgOff) +
                    static_cast<int64_t>((tile * S + slice) * P) * WORDS;  // the P parts of this (tile, slice)

  // The partial sums of one K part: x rows and A rows fetched row-contiguously (sixteen lanes per
  // 256 bytes of a row, unused rank blocks not at all), turned into
  // MFMA operand layout through the wavefront's LDS block, multiplied, and summed over the NWP
  // wavefronts in wavefront order.  tot[j] receives the sum of word tid + j * kNT.
  auto shrink_part = [&](int kp, float(&tot)[WPT]) {
    if (wave < NWP) {
      const int kcol = (kp * NWP + wave) * 128 + (lane & 15) * 8;  // first column of this lane's chunk
      i32x4 xst[4], ast[RB][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        xst[i] = load128(static_cast<const T*>(xv) + static_cast<int64_t>(rows4[i]) * xs + kcol);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int rr = rb * 16 + 4 * lg + i;
          if (RB == 1 || rb < rb_n) ast[rb][i] = load128(A + static_cast<int64_t>(rr < R ? rr : R - 1) * K + kcol);
        }
      }
      i32x4* stage = s_stage + wave * 16 * kStageRow;
      Pack8 xa[4], aw[4];
      f32x4 acc[RB];
#pragma unroll
      for (int i = 0; i < 4; ++i) stage[(4 * lg + i) * kStageRow + (lane & 15)] = xst[i];
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int i = 0; i < 4; ++i) xa[i].raw = stage[lr * kStageRow + 4 * i + lg];  // k-step i of lane group lg is chunk 4*i + lg
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (RB == 1 || rb < rb_n) {
#pragma unroll
          for (int i = 0; i < 4; ++i) stage[(4 * lg + i) * kStageRow + (lane & 15)] = ast[rb][i];
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int i = 0; i < 4; ++i) aw[i].raw = stage[lr * kStageRow + 4 * i + lg];
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[rb] = Mma<T>::run(xa[i], aw[i], acc[rb]);
        }
        // D layout: lane holds H[token 4*(lane/16)+i][rank 16*rb + lane%16]
        *reinterpret_cast<f32x4*>(&s_red[((wave * RB + rb) * 64 + lane) * 4]) = acc[rb];
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < WPT; ++j) {
      const int w = tid + j * kNT;  // word tok * R + r
      float sum = 0.f;
      if (WORDS % kNT == 0 || w < WORDS) {
        const int tok = w / R, r = w % R;
        const int idx = (((r >> 4) * 64) + (tok >> 2) * 16 + (r & 15)) * 4 + (tok & 3);
#pragma unroll
        for (int wv = 0; wv < NWP; ++wv) sum += s_red[wv * RB * 256 + idx];
      }
      tot[j] = sum;
    }
    __syncthreads();  // s_red may be rewritten by the next part
  };

  // ================================ consumer part: loads =========================================
  // ---- every load of the expand goes out first (before the shrink of a symmetric workgroup too) --
  const T* const Bs = static_cast<const T*>(sl.b[slice]) + static_cast<int64_t>(slot) * N * R;
  T* const ycols = static_cast<T*>(yv_) + sl.y_col[slice];
  const int eff8 = (eff + 7) >> 3;  // 8-rank chunks of a B row in use
  // span of 64 columns: MFMA j takes column c0 + 4 * (lane % 16) + j, so a lane ends up with four
  // consecutive columns of tokens 4 * (lane / 16) .. + 3
  auto load_span = [&](int c0, Pack8(&bo)[4][KSTEPS], uint2(&yy)[4]) {
    if constexpr (K16) {
      // A span's 64 B rows of 32 bytes are 2 KB of contiguous memory: fetched as such (lane l takes
      // 16 bytes of row c0 + l / 2 and of row c0 + 32 + l / 2); finish_span turns them into operand pieces.
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        int n = c0 + 32 * h + (lane >> 1);
        n = n < n1 ? n : n1 - 1;
        if ((lane & 1) < eff8) {
          bo[h][0].raw = load128(Bs + static_cast<int64_t>(n) * R + (lane & 1) * 8);
          if (eff & 7) mask_ranks(bo[h][0], (lane & 1) * 8, eff);
        } else {
          bo[h][0].raw = i32x4{0, 0, 0, 0};
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int n = c0 + 4 * lr + j;
        n = n < n1 ? n : n1 - 1;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const int kc = lg + 4 * ks;  // chunk of eight ranks this lane feeds to k-step ks
          if (kc < eff8) {
            bo[j][ks].raw = load128(Bs + static_cast<int64_t>(n) * R + kc * 8);
            if (eff & 7) mask_ranks(bo[j][ks], kc * 8, eff);
          } else {
            bo[j][ks].raw = i32x4{0, 0, 0, 0};
          }
        }
      }
    }
    const int c = c0 + 4 * lr < n1 ? c0 + 4 * lr : n1 - 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) yy[i] = *reinterpret_cast<const uint2*>(ycols + static_cast<int64_t>(rows4[i]) * ys + c);
  };
  Pack8 bop[kSpansAhead][4][KSTEPS];
  uint2 yq[kSpansAhead][4];
#pragma unroll
  for (int s = 0; s < kSpansAhead; ++s) {
    const int c0 = n0 + (wave + s * kNW) * 64;
    if (c0 < n1) load_span(c0, bop[s], yq[s]);
  }

  MLORA_STAMP(4);  // consumer: every load of the expand is issued
  // ================================ producer part ===============================================
  if (producer && xok) {
    float tot[WPT];
    shrink_part(part, tot);
    MLORA_STAMP(2);  // producer: its K part is multiplied and summed over the wavefronts
    u64* mine = xchg + part * WORDS;
#pragma unroll
    for (int j = 0; j < WPT; ++j) {
      const int w = tid + j * kNT;
      if ((WORDS % kNT == 0 || w < WORDS) && (w % R) < 16 * rb_n)
        xstore(mine + w, (static_cast<u64>(tag) << 32) | __float_as_uint(tot[j]), wide);
    }
    MLORA_STAMP(3);  // producer: partial sums handed to the memory system
  }
  if (!consumer || n0 >= n1) {  // nothing to expand here
    count_done();
    MLORA_STAMP(15);  // role marker: pure producers leave slot 15 non-zero
    return;
  }

  // ---- the intermediate: from the producers, or computed here ---------------------------------------
  // lane l of wavefront 0 takes words l * WPL .. + WPL - 1 (token l / 4, ranks (l % 4) * WPL ..) of every part
  if (wave == 0) {
    const int r0 = (lane & 3) * WPL;
    bool ok = xok;
    float sum[WPL];
    if (xok) {
      const long long t0 = wall_clock64();
      for (;;) {
        bool all = true;
#pragma unroll
        for (int q = 0; q < WPL; ++q) sum[q] = 0.f;
        for (int kp = 0; kp < P; ++kp) {
          u64 v[WPL];
#pragma unroll
          for (int q = 0; q < WPL; ++q) v[q] = (r0 + q < 16 * rb_n) ? xload(xchg + kp * WORDS + lane * WPL + q, wide) : (static_cast<u64>(tag) << 32);
#pragma unroll
          for (int q = 0; q < WPL; ++q) {
            all &= static_cast<uint32_t>(v[q] >> 32) == tag;
            sum[q] += __uint_as_float(static_cast<uint32_t>(v[q]));
          }
        }
        ok = spin_ticks >= 0 && __builtin_amdgcn_ballot_w64(all) == ~0ull;
        if (ok || wall_clock64() - t0 >= spin_ticks) break;
        if (!(wide & 32)) __builtin_amdgcn_s_sleep(1);
        if (wide & 8) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // drop what the L1 holds of the polled lines
        if (wide & 16) asm volatile("buffer_inv sc0" ::: "memory");        // the same, this compute unit's L1 only
      }
      if (!ok && spin_ticks > 0 && lane == 0) atomicAdd(ws + kWsTimeoutsWord, 1u);  // diagnostic: a wait ran out
    }
    if (ok) {
      const int tok = lane >> 2;
#pragma unroll
      for (int q = 0; q < WPL; ++q) {
        const int r = r0 + q;
        const float v = r < eff ? sum[q] * scaling : 0.f;  // ranks the adapter does not have contribute nothing
        const T hi = from_f32<T>(v);
        s_hi[tok * HSTRIDE + r] = hi;
        s_lo[tok * HSTRIDE + r] = from_f32<T>(v - to_f32(hi));
      }
    }
    if (lane == 0) s_ok = ok;
    MLORA_STAMP(5);  // consumer: the wait for the producers is over
  }
  __syncthreads();
  if (!s_ok) {
    // every part computed here, added up in the order the consumers of published parts use
    float total[WPT];
#pragma unroll
    for (int j = 0; j < WPT; ++j) total[j] = 0.f;
    for (int kp = 0; kp < P; ++kp) {
      float tot[WPT];
      shrink_part(kp, tot);
#pragma unroll
      for (int j = 0; j < WPT; ++j) total[j] += tot[j];
    }
#pragma unroll
    for (int j = 0; j < WPT; ++j) {
      const int w = tid + j * kNT;
      if (WORDS % kNT == 0 || w < WORDS) {
        const int tok = w / R, r = w % R;
        const float v = r < eff ? total[j] * scaling : 0.f;
        const T hi = from_f32<T>(v);
        s_hi[tok * HSTRIDE + r] = hi;
        s_lo[tok * HSTRIDE + r] = from_f32<T>(v - to_f32(hi));
      }
    }
    __syncthreads();
    // the expand's operands are requested again rather than kept in registers across the shrink
    // (this path is the exception; the registers it would cost are paid by every launch)
#pragma unroll
    for (int s = 0; s < kSpansAhead; ++s) {
      const int c0 = n0 + (wave + s * kNW) * 64;
      if (c0 < n1) load_span(c0, bop[s], yq[s]);
    }
  }
  count_done();  // this workgroup reads the exchange area no more
  MLORA_STAMP(6);  // consumer: the intermediate is in LDS, the arrival counted

  // ---- expand ---------------------------------------------------------------------------------------
  Pack8 hop[KSTEPS], hlo[KSTEPS];
  uint2 hop16 = {0, 0}, hlo16 = {0, 0};
  if constexpr (K16) {
    hop16 = *reinterpret_cast<const uint2*>(&s_hi[lr * HSTRIDE + 4 * lg]);
    hlo16 = *reinterpret_cast<const uint2*>(&s_lo[lr * HSTRIDE + 4 * lg]);
  } else {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const int kc = lg + 4 * ks;
      if (kc * 8 < R) {
        hop[ks].raw = load128(&s_hi[lr * HSTRIDE + kc * 8]);
        hlo[ks].raw = load128(&s_lo[lr * HSTRIDE + kc * 8]);
      } else {
        hop[ks].raw = i32x4{0, 0, 0, 0};
        hlo[ks].raw = i32x4{0, 0, 0, 0};
      }
    }
  }
  const int ks_n = (eff + 31) >> 5;  // k-steps of the expand in use
  // tokens as MFMA rows: lane holds out[token 4 * lg + i][column c0 + 4 * lr + j]
  auto finish_span = [&](int c0, Pack8(&bo)[4][KSTEPS], uint2(&yy)[4]) {
    f32x4 out[4];
    uint2 pieces[4];
    if constexpr (K16) {
      // B rows -> operand pieces through the wavefront's LDS block: four rows (128 bytes) per
      // group, groups 144 bytes apart so that the sixteen lanes of a piece read hit every bank
      // once.  MFMA j of lane (lr, lg) takes ranks 4*lg .. 4*lg+3 of column c0 + 4*lr + j.
      char* blk = reinterpret_cast<char*>(s_stage + wave * 16 * kStageRow);
      *reinterpret_cast<i32x4*>(blk + (lane >> 3) * 144 + (lane & 7) * 16) = bo[0][0].raw;
      *reinterpret_cast<i32x4*>(blk + ((lane >> 3) + 8) * 144 + (lane & 7) * 16) = bo[1][0].raw;
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < 4; ++j) pieces[j] = *reinterpret_cast<const uint2*>(blk + lr * 144 + j * 32 + lg * 8);
      __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      out[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      if constexpr (K16) {
        const uint2 piece = pieces[j];
        out[j] = Mma16<T>::run(hlo16, piece, out[j]);
        out[j] = Mma16<T>::run(hop16, piece, out[j]);
      } else {
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          if (KSTEPS == 1 || ks < ks_n) {
            out[j] = Mma<T>::run(hlo[ks], bo[j][ks], out[j]);
            out[j] = Mma<T>::run(hop[ks], bo[j][ks], out[j]);
          }
        }
      }
    }
    if constexpr (!K16 && KSTEPS > 1) mfma_settle(out);  // k-steps beyond the adapter's rank were skipped by branches
    const int c = c0 + 4 * lr;
    if (c < n1) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (4 * lg + i < m) {
          union { uint2 raw; T e[4]; } v;
          v.raw = yy[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) v.e[j] = from_f32<T>(to_f32(v.e[j]) + out[j][i]);
          *reinterpret_cast<uint2*>(ycols + static_cast<int64_t>(rows4[i]) * ys + c) = v.raw;
        }
      }
    }
  };
#pragma unroll
  for (int s = 0; s < kSpansAhead; ++s) {
    const int c0 = n0 + (wave + s * kNW) * 64;
    if (c0 < n1) finish_span(c0, bop[s], yq[s]);
  }
  MLORA_STAMP(7);  // consumer, wavefront 0: its first spans are multiplied and their stores issued
  for (int c0 = n0 + (wave + kSpansAhead * kNW) * 64; c0 < n1; c0 += kNW * 64) {  // wide ranges
    Pack8 bo[4][KSTEPS];
    uint2 yt[4];
    load_span(c0, bo, yt);
    finish_span(c0, bo, yt);
  }
#ifdef MLORA_TRACE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  MLORA_STAMP(8);  // wavefront 0: its stores are acknowledged
  __syncthreads();
  MLORA_STAMP(9);  // every wavefront is done
#endif
}

// Clears the head of a workspace (tile generations, arrival counts, exchange area) and writes
// the signature.
__global__ __launch_bounds__(256) void workspace_init_kernel(uint32_t* ws) {
  const int words = MLORA_WORKSPACE_HEAD_BYTES / 4;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < words; i += gridDim.x * blockDim.x)
    ws[i] = i == 0 ? kWsMagic : i == kWsTileOff / 4 + 2 ? kWsGenCheck : 0u;  // generation 0 and its check word
}

struct SplitLaunch {
  const MloraAddArgs* a;
  dim3 grid;
  int small_off, include_long, S, P, W, spin_ticks, wide, trusted, sym;
  SplitSlices sl;
};

template <typename T, int R, int NWP, bool MASKED>
void launch_split_masked(const SplitLaunch& l) {
  const MloraAddArgs* a = l.a;
  hipLaunchKernelGGL((split_kernel<T, R, NWP, MASKED>), l.grid, dim3(kNT), 0, static_cast<hipStream_t>(a->stream), a->plan, a->x, a->y, a->x_stride,
                     a->y_stride, static_cast<uint32_t*>(a->workspace), l.small_off, a->num_tokens, a->k, a->num_slots, a->scaling,
                     l.include_long, l.S, l.P, l.W, l.spin_ticks, l.wide, l.trusted, l.sym, a->effective_rank, l.sl);
}

// With a rank vector the instance that reads it; without, the one that has no such code at all.
template <typename T, int R, int NWP>
void launch_split_one(const SplitLaunch& l) {
  if (l.a->effective_rank) launch_split_masked<T, R, NWP, true>(l);
  else launch_split_masked<T, R, NWP, false>(l);
}

template <typename T>
void launch_split_rank(const SplitLaunch& l, int nwp) {
#define MLORA_SPLIT(R_)                                              \
  if (nwp == 8) launch_split_one<T, R_, 8>(l);                       \
  else launch_split_one<T, R_, 4>(l)
  switch (l.a->r) {
    case 8: MLORA_SPLIT(8); break;
    case 16: MLORA_SPLIT(16); break;
    case 32: MLORA_SPLIT(32); break;
    default: MLORA_SPLIT(64); break;
  }
#undef MLORA_SPLIT
}

// Diagnostic knobs, read from the environment once per process.
struct SplitKnobs {
  int generation = -1, w, spin_ticks, wide, kpart, sym;
  void read() {
    generation = knob_generation();
    w = env_int("MLORA_SPLIT_W", 0);
    spin_ticks = env_int("MLORA_SPLIT_SPIN_TICKS", 20000);  // 200 us of the 100 MHz clock; negative: never accept published sums
    // loads and the arrival counts at device scope, stores in the L2 of the XCD on which every
    // workgroup of a tile runs: were a tile ever spread over XCDs, its consumers would not see the
    // stores, give up waiting and compute for themselves, and the generations would still advance
    wide = env_int("MLORA_SPLIT_WIDE", 5);
    sym = env_int("MLORA_SPLIT_SYM", -1);    // -1: symmetric roles when a tile's shrink has four or more K parts
    kpart = env_int("MLORA_SPLIT_KPART", 0);
  }
};

}  // namespace

void split_trace_set(void* buf) {
#ifdef MLORA_TRACE
  (void)hipMemcpyToSymbol(HIP_SYMBOL(trace_buf), &buf, sizeof(buf));
#else
  (void)buf;
#endif
}

int workspace_init(void* workspace, hipStream_t stream) {
  hipLaunchKernelGGL(workspace_init_kernel, dim3(256), dim3(256), 0, stream, static_cast<uint32_t*>(workspace));
  return check_launch("mlora_workspace_init");
}

// Columns of a K part: 1024 (eight wavefronts) when K is long, 512 (four) otherwise, so that a
// producer pulls 24-48 KB and a consumer adds up at most eight parts; the other width when the
// preferred one does not divide K or its partial sums do not fit the exchange area.  0: none fits.
static int pick_kpart(const MloraAddArgs* a, int wanted) {
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  const int preferred = (a->k % 1024 == 0 && a->k >= 2048) ? 1024 : 512;
  const int order[3] = {wanted, preferred, preferred == 512 ? 1024 : 512};
  for (int kp : order) {
    if (kp != 512 && kp != 1024) continue;
    if (a->k % kp != 0 || a->k / kp > 8) continue;
    if (static_cast<int64_t>(lay.cap_small) * a->num_slices * (a->k / kp) * 16 * a->r * 8 <= kWsXchgBytes) return kp;
  }
  return 0;
}

// Whether the split form can take this call at all (shape, workspace, partial sums that fit the
// exchange area).
bool split_supported(const MloraAddArgs* a) {
  if (!a->workspace || (reinterpret_cast<uintptr_t>(a->workspace) & 255) || a->workspace_bytes < MLORA_WORKSPACE_HEAD_BYTES) return false;
  if (a->k % 512 != 0 || a->k < 512 || !exact_rank(a->r)) return false;
  if (plan_layout(a->num_tokens, a->num_slots).cap_small > kWsTiles) return false;
  for (int i = 0; i < a->num_slices; ++i)
    if (a->slices[i].n <= 0) return false;
  return pick_kpart(a, 0) != 0;
}

int launch_split(const MloraAddArgs* a, bool include_long, bool trusted_workspace) {
  static SplitKnobs knobs;
  if (knobs.generation != knob_generation()) knobs.read();
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  int cap = lay.cap_small;
  if (!include_long) {  // a segment below the threshold is exactly one small tile
    const int segs = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;
    if (segs < cap) cap = segs;
  }
  if (cap == 0) return 0;
  cap = (cap + 7) & ~7;

  SplitLaunch l;
  l.a = a; l.small_off = lay.small_off; l.include_long = include_long ? 1 : 0;
  l.S = a->num_slices;
  l.spin_ticks = knobs.spin_ticks; l.wide = knobs.wide; l.trusted = trusted_workspace ? 1 : 0;
  const int kp = pick_kpart(a, knobs.kpart);  // split_supported() was true: some width fits
  l.P = a->k / kp;
  const int nwp = kp / 128;

  // Column range of a consumer: so that the launch has about 512 consumers (two per compute
  // unit), between 128 and 1024 columns (a wavefront holds the loads of two 64-column spans)
  long long cols = 0;
  for (int i = 0; i < a->num_slices; ++i) cols += a->slices[i].n;
  int w = knobs.w;
  if (w <= 0) {
    const int segs = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;
    const int by_tokens = (a->num_tokens + MLORA_TILE_SMALL - 1) / MLORA_TILE_SMALL;
    const long long tiles = segs > by_tokens ? segs : by_tokens;  // about the number of tiles in use
    w = static_cast<int>(cols * tiles / 512);
    if (w > 1024) w = 1024;
    if (w < 128) w = 128;
  }
  w = (w + 63) & ~63;
  int consumers = 0;
  for (int i = 0; i < MLORA_MAX_SLICES; ++i) {
    l.sl.cons0[i] = consumers;
    if (i < a->num_slices) {
      const MloraSlice& s = a->slices[i];
      l.sl.a[i] = s.a; l.sl.b[i] = s.b; l.sl.n[i] = s.n; l.sl.y_col[i] = s.y_col;
      consumers += (s.n + w - 1) / w;
    } else {
      l.sl.a[i] = nullptr; l.sl.b[i] = nullptr; l.sl.n[i] = 0; l.sl.y_col[i] = 0;
    }
  }
  l.sl.cons0[MLORA_MAX_SLICES] = consumers;
  l.W = w;
  l.sym = knobs.sym >= 0 ? (knobs.sym ? 1 : 0) : (l.P >= 4 ? 1 : 0);
  // producers first: they are dispatched before the consumers that wait for them
  l.grid = dim3(8, static_cast<unsigned>(l.sym ? l.S * l.P : l.S * l.P + consumers), static_cast<unsigned>(cap / 8));
  if (a->dtype == MLORA_DTYPE_BF16) launch_split_rank<__bf16>(l, nwp);
  else launch_split_rank<_Float16>(l, nwp);
  return check_launch("mlora_add_lora(small tiles, producers and consumers)");
}

}  // namespace mlora
